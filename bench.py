#!/usr/bin/env python3
"""Benchmark of the mesh-conv hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload scene|shapes|pool|firstblock|tail|hierarchy|texture|pcloud|decimate] [--scale S]

A step is one forward+backward pass of the layer over one batch of seeded synthetic meshes
already resident in HBM.  Default workload ``scene``: 8 room-like meshes of about 300 k
facets each, texture points per facet 1..9 by area, F2F (64 -> 64, SH degree 3) followed by
F2V (64 -> 64) in float32, gradient dL/dy ~ N(0,1) -- the native ops only; the pointwise
matmul / bias / ReLU / batch-norm tail of the modules is ordinary PyTorch and not timed.

Prints ONE JSON line with the whole-job throughput in Mfacets/s, the roofline figure of the
dominant kernel (HIP events on the launch stream, inside the timed region) and the CPU
baseline (the vectorised oracle in float32 on the host cores, on a bounded sample).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F32_PEAK_TFLOPS = 157.3
MFMA_F16_PEAK_TFLOPS = 2500.0
# The facet2facet kernels get fp32 accuracy from three fp16 piece products per product (two-piece split of both
# operands), so the matrix-core ceiling for their algorithmic (fp32-equivalent) flops is a third of the fp16 peak.
F2F_PIECE_PRODUCTS = 3


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="scene", choices=["scene", "shapes", "pool", "firstblock", "tail", "f2vtail", "hierarchy", "texture", "pcloud", "decimate"],
                    help="scene: the headline layer (F2F+F2V, C=64); shapes: 16 small meshes V2F+F2F+F2V; pool: "
                         "1024x1024 grid max/avg pool + unpool; firstblock: the scene batch with the reference's first "
                         "block shapes, F2F 3->32 then F2V 32->32 with depth multiplier 2 (pi2_blocks.py:113-130)")
    ap.add_argument("--scale", type=float, default=1.0, help="facet-count scale of the scene workload")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--degree", type=int, default=3, choices=[0, 1, 2, 3, 4, 5],
                    help="spherical-harmonic degree of the scene workload's filters (3 = the headline configuration)")
    ap.add_argument("--f2f-half", action="store_true",
                    help="facet2facet in its half-precision variant (one fp16 piece per operand, fp32 accumulation; "
                         "results within 1e-3 instead of 1e-5): a separate figure, never the default")
    ap.add_argument("--bf16-features", action="store_true",
                    help="scene workload with the features (texture rows, layer outputs, their gradients) kept in bf16 "
                         "in HBM and one fp16 product per element with fp32 accumulation: a separate figure")
    ap.add_argument("--graph", action="store_true",
                    help="hierarchy workload: also record the step (forward + backward) once as a HIP graph and time its replays")
    ap.add_argument("--traffic-from", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no benchmark: turn the counter_collection CSVs of two rocprofv3 --pmc runs (FETCH_SIZE, "
                         "WRITE_SIZE) of this workload into profiles/traffic.json and a text summary")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="after the timed region, copy a 1 GiB buffer three times (a kernel of known HBM traffic "
                         "to scale rocprofv3's FETCH_SIZE / WRITE_SIZE counters by)")
    return ap.parse_args()


# ---------------------------------------------------------------------------- inputs
def build_conv_inputs(mesh, C, L, seed, tex_counts="area", Cin=None, r=1):
    from picassoplus_amd import synthetic as S
    rng = np.random.default_rng(seed)
    v, f = mesh["vertex"], mesh["face"]
    nv, nf = v.shape[0], f.shape[0]
    normal, area = S.triangle_normals_areas(v, f)
    counts = S.area_scaled_texture_counts(area) if tex_counts == "area" else np.full(nf, int(tex_counts), np.int32)
    counts, bary, owner = S.texture_points(rng, nf, counts)
    B = (L + 1) ** 2
    return dict(
        nv=nv, nf=nf, T=int(counts.sum()), C=C, Cin=Cin or C, r=r, B=B, L=L, face=f, normal=normal.astype(np.float32),
        counts=counts, bary=bary.astype(np.float32), owner=owner,
        vt_map=np.arange(nv, dtype=np.int32), nf_count=np.maximum(S.vertex_facet_count(f, np.arange(nv), nv), 1),
        x=rng.uniform(-1, 1, (nv, C)).astype(np.float32),
        w_f2f=S.xavier_uniform(rng, (C, Cin or C, B), (Cin or C) * B, C * B).astype(np.float32),
        w_f2v=S.xavier_uniform(rng, (B, C, r), C, B * C * r).astype(np.float32),
        w_v2f=S.xavier_uniform(rng, (3, C, 1), C, 3 * C).astype(np.float32),
        mf_in=mesh["mf_in"], nv_in=mesh["nv_in"])


def conv_bytes_flops(d, ops, fb=4):
    """Algorithmic HBM bytes / flops per op: every input read once, every output written once.  ``fb`` = bytes per
    FEATURE value (texture rows, layer inputs / outputs and their gradients): 4, or 2 for the bf16-feature variant;
    indices, SH coefficients, filters and filter gradients are 4 bytes in both."""
    Nf, Nv, T, C, B = d["nf"], d["nv"], d["T"], d["C"], d["B"]
    Ci, r = d["Cin"], d["r"]                    # F2F input channels; F2V depth multiplier (output width C * r)
    tab = {
        "v2f_fwd": (fb * Nv * C + 12 * Nf + fb * Nf * C, 6 * Nf * C),
        "v2f_bwd": (fb * Nf * C + 12 * Nf + 2 * fb * Nv * C, 12 * Nf * C),
        "f2v_fwd": (fb * Nf * C + 4 * Nf * B + 12 * Nf + 8 * Nv + fb * Nv * C * r, Nf * C * r * (2 * B + 7)),
        "f2v_bwd": (fb * Nv * C * r + 2 * fb * Nf * C + 4 * Nf * B + 12 * Nf + 8 * Nv, Nf * C * r * (4 * B + 12)),
        "f2f_fwd": (fb * T * Ci + 4 * T * B + 4 * Nf + 4 * C * Ci * B + fb * Nf * C, 2 * T * Ci * B + 2 * Nf * Ci * B * C),
        "f2f_bwd_texture": (fb * Nf * C + 4 * T * B + 4 * Nf + 4 * C * Ci * B + fb * T * Ci, 2 * Nf * Ci * B * C + 2 * T * Ci * B),
        "f2f_bwd_filter": (fb * Nf * C + fb * T * Ci + 4 * T * B + 4 * Nf + 4 * C * Ci * B, 2 * Nf * Ci * B * C + 2 * T * Ci * B),
        # texture points interpolated from vertex features, with their basis values (forward) / transposed (backward)
        "texture_fwd": (4 * Nv * C + 16 * Nf + 12 * T + 4 * T * C + 4 * T * B, 5 * T * C + 60 * T),
        "texture_bwd": (4 * T * C + 12 * T + 16 * Nf + 4 * Nv * C, 6 * T * C),
    }
    return {k: tab[k] for k in ops}


# ---------------------------------------------------------------------------- measured HBM traffic
# roofline.traffic = HBM bytes per launch of the dominant op from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per
# dispatch), scaled by what the same counters read for a 1 GiB device copy (--copy-calibration).  The figures live in
# profiles/traffic.json, written by `bench.py --traffic-from FETCH.csv WRITE.csv --workload W` from the two counter
# runs, together with the identity of the build they were measured on (a hash over the kernel sources): a bench run
# of any other build reports traffic = null instead of a stale number.
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "traffic.json")
# op -> kernels whose traffic it sums (regular expressions on the demangled kernel name, after "pmesh::")
TRAFFIC_KERNELS = {
    "scene": {"f2f_fwd": [r"f2f16h2_fwd_k"], "f2f_bwd_texture": [r"f2f16h2_bwd_tex_k"],
              "f2f_bwd_filter": [r"f2f16h2_bwd_filt_k", r"f2f16x3_bwd_filt_k", r"f2f_reduce_k"],
              "f2v_fwd": [r"f2v_fwd_mfma_k"], "f2v_bwd": [r"f2v_bwd_mfma_k", r"reduce_partials_k"]},
    "pool": {"pool_max_fwd": [r"pool_max_fwd_k"], "pool_max_bwd": [r"fine_gather_k<4, 2>"],
             "pool_avg_fwd": [r"cluster_sum_k<4, true>"], "pool_avg_bwd": [r"fine_gather_k<4, 1>"],
             "unpool_fwd": [r"fine_gather_k<4, 0>"], "unpool_bwd": [r"cluster_sum_k<4, false>"]},
    "tail": {"dense_fwd": [r"dense_rows_k<\d+, \d+, (true|false), 0, "],
             "dense_bwd": [r"dense_rows_k<\d+, \d+, (true|false), [12], ", r"dense_wgrad_k", r"reduce_partials_k"]},
    "texture": {"texture_fwd": [r"texture_fwd_k"], "texture_bwd": [r"texture_bwd_flat_k", r"texture_bwd_k"]},
    "pcloud": {"point_conv_fwd": [r"point_conv_rows_dense_k<\d+, 0>", r"point_conv_fwd_k"],
               "point_conv_bwd": [r"point_conv_bwd_fused_k", r"point_conv_rows_dense_k<\d+, 1>", r"point_conv_bwd_in_k", r"point_conv_bwd_filt", r"reduce_partials_k"]},
}


def build_id():
    """Identity of the kernels being timed: hash over every source of the native library (kernels of all workloads,
    the index builds, neighbour searches and mesh preparation included, and their shared headers)."""
    import hashlib
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "picassoplus_amd", "csrc")
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".h", ".cpp")):
            h.update(name.encode())
            h.update(open(os.path.join(csrc, name), "rb").read())
    return h.hexdigest()[:16]


def measured_traffic(workload, variant, op):
    """Bytes per launch of `op` from profiles/traffic.json, or None when the file is absent, holds another build's
    figures or does not cover this workload variant."""
    try:
        tab = json.load(open(TRAFFIC_JSON))
    except (OSError, ValueError):
        return None
    ent = tab.get(workload + ("+" + variant if variant else ""))
    if not ent or ent.get("build_id") != build_id():
        return None
    return ent.get("bytes_per_launch", {}).get(op)


def write_traffic(args):
    """profiles/traffic.json (and a text summary beside it) from the two rocprofv3 counter runs of one workload."""
    import csv, re, subprocess
    def agg(path, counter):
        out = {}
        for r in csv.DictReader(open(path)):
            if r["Counter_Name"] == counter:
                name = re.sub(r"^void ", "", r["Kernel_Name"])
                name = re.sub(r"\(.*$", "", name)
                out.setdefault(name, []).append(float(r["Counter_Value"]))
        return out
    F, W = agg(args.traffic_from[0], "FETCH_SIZE"), agg(args.traffic_from[1], "WRITE_SIZE")
    copy = [k for k in F if "copyBuffer" in k]
    if not copy or copy[0] not in W:
        sys.exit("--traffic-from: no device-copy kernel in the counter files (run bench.py with --copy-calibration)")
    # the three 1 GiB copies are the copy kernel's three largest dispatches
    fcal, wcal = sum(sorted(F[copy[0]])[-3:]) / 3.0, sum(sorted(W[copy[0]])[-3:]) / 3.0
    ff, wf = 1048576.0 / fcal, 1048576.0 / wcal
    per_kernel, ops = {}, {}
    for op, pats in TRAFFIC_KERNELS[args.workload].items():
        tot = 0.0
        for pat in pats:
            for k in sorted(set(F) | set(W)):
                short = k.replace("pmesh::", "")
                if re.match(pat, short) or re.search(pat, short):
                    f = sum(F.get(k, [0])) / max(len(F.get(k, [0])), 1)
                    w = sum(W.get(k, [0])) / max(len(W.get(k, [0])), 1)
                    per_kernel[short] = (f, w, f * 1024 * ff, w * 1024 * wf)
                    tot += f * 1024 * ff + w * 1024 * wf
        ops[op] = tot
    key = args.workload + ("+f2f-half" if args.f2f_half else "") + ("+bf16" if args.bf16_features else "")
    try:
        tab = json.load(open(TRAFFIC_JSON))
    except (OSError, ValueError):
        tab = {}
    try:
        git = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True).stdout.strip()
    except OSError:
        git = ""
    tab[key] = dict(build_id=build_id(), git_head_when_measured=git, scale_fetch=ff, scale_write=wf,
                    bytes_per_launch={k: round(v) for k, v in ops.items()})
    json.dump(tab, open(TRAFFIC_JSON, "w"), indent=1, sort_keys=True)
    lines = ["HBM traffic per launch from rocprofv3 PMC, workload %s, MI355X, build %s" % (key, build_id()),
             "commands (from /tmp, TMPDIR=/tmp), one counter per run, then the summary:",
             "  rocprofv3 --pmc FETCH_SIZE -d <out> -o pmc --output-format csv -- python3 bench.py --workload %s --steps 2 --warmup 1 --no-cpu-baseline --copy-calibration" % args.workload,
             "  rocprofv3 --pmc WRITE_SIZE -d <out> -o pmc --output-format csv -- python3 bench.py --workload %s --steps 2 --warmup 1 --no-cpu-baseline --copy-calibration" % args.workload,
             "  python3 bench.py --workload %s --traffic-from <FETCH csv> <WRITE csv>" % args.workload,
             "calibration: three 1 GiB device copies read %.0f KiB (FETCH_SIZE) and %.0f KiB (WRITE_SIZE) per copy -> scale factors %.3f and %.3f" % (fcal, wcal, ff, wf), "",
             "%-44s %14s %14s %10s %10s" % ("kernel (mean per launch)", "FETCH_SIZE KiB", "WRITE_SIZE KiB", "read GB", "written GB")]
    for k, (f, w, rb, wb) in per_kernel.items():
        lines.append("%-44s %14.1f %14.1f %10.3f %10.3f" % (k[:44], f, w, rb / 1e9, wb / 1e9))
    lines += ["", "per op (sum of its kernels), as written to profiles/traffic.json:"]
    lines += ["  %-18s %.3f GB" % (k, v / 1e9) for k, v in ops.items()]
    out = os.path.join(ROOT, "profiles", "%s_hbm_traffic_pmc.txt" % key.replace("+", "_"))
    open(out, "w").write("\n".join(lines) + "\n")
    print("\n".join(lines))


class EventTimer:
    """Brackets every native call with HIP events on the launch stream."""

    def __init__(self, torch):
        self.torch, self.open, self.pairs, self.on = torch, {}, [], False

    def __call__(self, name, phase):
        if not self.on:
            return
        ev = self.torch.cuda.Event(enable_timing=True)
        ev.record()
        if phase == "begin":
            self.open[name] = ev
        else:
            self.pairs.append((name, self.open.pop(name), ev))

    def summary(self):
        tot, cnt = {}, {}
        for name, a, b in self.pairs:
            key = name.replace("pmesh_", "")
            tot[key] = tot.get(key, 0.0) + a.elapsed_time(b)
            cnt[key] = cnt.get(key, 0) + 1
        return {k: tot[k] / cnt[k] for k in tot}

    def totals(self, steps):
        """Milliseconds per step and entry point, summed over all of a step's calls."""
        tot = {}
        for name, a, b in self.pairs:
            key = name.replace("pmesh_", "")
            tot[key] = tot.get(key, 0.0) + a.elapsed_time(b)
        return {k: v / steps for k, v in tot.items()}


# ---------------------------------------------------------------------------- workloads
def run_conv_layer(args, torch, kind):
    from picassoplus_amd import _lib, synthetic as S
    from picassoplus_amd.mesh.layers import sph_harm_values
    from picassoplus_amd.mesh.pi_modules import conv3d, texture
    dev = torch.device("cuda:0")
    C, L = (32 if kind == "firstblock" else 64), 3           # first block: EncodeChannels[0] = 32 (scene_seg.py:28)
    if args.degree != 3:
        if kind != "scene":
            sys.exit("--degree is a variant of the scene workload")
        L = args.degree
    Cin, r = (3, 2) if kind == "firstblock" else (C, 1)      # F2F input channels, F2V depth multiplier
    if kind in ("scene", "firstblock"):
        mesh = S.scene_workload(seed=3000, n_rooms=8, scale=args.scale)
        d = build_conv_inputs(mesh, C, L, seed=3000, Cin=Cin, r=r)
        ops = ["f2f_fwd", "f2v_fwd", "f2v_bwd", "f2f_bwd_texture", "f2f_bwd_filter"]
        name = "scene8x300k_F2F+F2V_C64_L%d_fp32_fwd+bwd" % L if kind == "scene" else "scene8x300k_F2F3to32+F2V32r2_L3_fp32_fwd+bwd"
    else:
        mesh = S.shapes_workload(seed=2000, n_meshes=16)
        d = build_conv_inputs(mesh, C, L, seed=2000, tex_counts=3)
        ops = ["v2f_fwd", "texture_fwd", "f2f_fwd", "f2v_fwd", "f2v_bwd", "f2f_bwd_texture", "f2f_bwd_filter",
               "texture_bwd", "v2f_bwd"]
        name = "shapes16_V2F+texture+F2F+F2V_C64_L3_fp32_fwd+bwd"
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    face, vt_map, nfc = t(d["face"]), t(d["vt_map"]), t(d["nf_count"].astype(np.int32))
    cum = torch.cumsum(t(d["counts"]), 0, dtype=torch.int32)
    bary = t(d["bary"])
    owner = t(d["owner"])
    x = t(d["x"])
    # scene workloads take the texture-point features as given data, like the reference's networks (set-up, untimed);
    # the shapes block interpolates them from the vertex features inside the step
    tex, sh = texture.interpolate(x, face, bary, cum, L)
    tex = tex[:, :Cin].contiguous()                          # first block: three colour-like channels
    del owner
    coeff = sph_harm_values(t(d["normal"]), L)
    w_f2f, w_f2v, w_v2f = t(d["w_f2f"]), t(d["w_f2v"]), t(d["w_v2f"])
    gy = torch.randn(d["nv"], C * r, device=dev, generator=torch.Generator(device=dev).manual_seed(1))
    bf16 = bool(args.bf16_features)
    if bf16:
        if kind != "scene":
            sys.exit("--bf16-features is a variant of the scene workload")
        tex, gy = tex.to(torch.bfloat16), gy.to(torch.bfloat16)
        name = "scene8x300k_F2F+F2V_C64_L3_bf16-features_fwd+bwd"
    tex.requires_grad_(True); w_f2f.requires_grad_(True); w_f2v.requires_grad_(True)
    if kind == "shapes":
        x.requires_grad_(True); w_v2f.requires_grad_(True)

    def step():
        if kind in ("scene", "firstblock"):
            y1 = conv3d.facet2facet(tex, w_f2f, sh, cum)
            y = conv3d.facet2vertex(y1, w_f2v, coeff, face, nfc, vt_map)
            return torch.autograd.grad(y, [tex, w_f2f, w_f2v], gy)
        y0 = conv3d.vertex2facet(x, w_v2f, face)
        tex_s, sh_s = texture.interpolate(x, face, bary, cum, L)
        y1 = conv3d.facet2facet(tex_s, w_f2f, sh_s, cum)
        y = conv3d.facet2vertex(y0 + y1, w_f2v, coeff, face, nfc, vt_map)
        return torch.autograd.grad(y, [x, w_v2f, w_f2f, w_f2v], gy)

    timer = EventTimer(torch)
    _lib.set_call_hook(timer)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer.on = True
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    timer.on = False
    _lib.set_call_hook(None)
    ms = (t1 - t0) * 1e3 / args.steps
    # per entry point and step (a degree other than 3 calls an entry point once per block of 16 coefficients)
    per_op = {k.replace("_bf16", ""): v for k, v in timer.totals(args.steps).items()}
    bf = conv_bytes_flops(d, ops, 2 if bf16 else 4)
    total_bytes = sum(b for b, _ in bf.values())
    dom = max(ops, key=lambda k: per_op.get(k, 0.0))
    dom_ms = per_op[dom]
    if dom.startswith("f2f") and Cin >= 16:
        ach = bf[dom][1] / (dom_ms * 1e-3) / 1e12
        pieces = 1 if (args.f2f_half or bf16) else F2F_PIECE_PRODUCTS
        roof = dict(bound="mfma", achieved=ach, peak=MFMA_F16_PEAK_TFLOPS / pieces, unit="TFLOP/s",
                    peak_basis="fp16 dense MFMA 2500 TFLOP/s, one product per element (reduced-precision variant)" if pieces == 1
                    else "fp16 dense MFMA 2500 TFLOP/s / 3 piece products per fp32-accurate product",
                    frac_of_fp32_mfma_peak=ach / MFMA_F32_PEAK_TFLOPS)
    else:
        roof = dict(bound="hbm", achieved=bf[dom][0] / (dom_ms * 1e-3) / 1e9, peak=HBM_PEAK_GBS, unit="GB/s")
    traffic = (measured_traffic("scene", "bf16" if bf16 else "f2f-half" if args.f2f_half else "", dom)
               if (kind == "scene" and args.scale == 1.0 and L == 3) else None)
    roof.update(frac=roof["achieved"] / roof["peak"], traffic=traffic, kernel=dom, kernel_ms=dom_ms)
    # adjacency of the step's index tensors, built cold (fresh tensors, nothing cached, range checks included): what
    # a training loop that gets new index tensors with every batch pays per step on top of ms_per_step
    from picassoplus_amd.mesh import topology
    index_ms = {}
    for label, build in (("vertex_csr", lambda: topology.vertex_csr(face.clone(), vt_map.clone(), d["nv"])),
                         ("facet_order", lambda: topology.facet_order(cum.clone(), d["T"]))):
        best = None
        for _ in range(3):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            build()
            torch.cuda.synchronize()
            dt = (time.perf_counter() - t0) * 1e3
            best = dt if best is None else min(best, dt)
        index_ms[label] = best
    if kind == "shapes":
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        topology.vertex_csr(face.clone(), None, d["nv"])
        torch.cuda.synchronize()
        index_ms["vertex_csr_inputs"] = (time.perf_counter() - t0) * 1e3
    ops_report = {k: dict(ms=per_op.get(k), gbps=bf[k][0] / (per_op[k] * 1e-3) / 1e9,
                          tflops=bf[k][1] / (per_op[k] * 1e-3) / 1e12) for k in ops if k in per_op}
    res = dict(value=d["nf"] / (ms * 1e-3) / 1e6, ms_per_step=ms, roofline=roof, ops=ops_report,
               hbm_gbps=total_bytes / (ms * 1e-3) / 1e9, hbm_frac=total_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
               index_build_ms=sum(index_ms.values()), index_build=index_ms,
               dtype=("bf16 features in HBM (texture rows, layer outputs, their gradients), f32 filters and coefficients; "
                      "facet2facet products one fp16 piece per operand on v_mfma_f32_32x32x16_f16, every sum accumulated in f32"
                      if bf16 else
                      "f32 in HBM; facet2facet products one fp16 piece per operand on v_mfma_f32_32x32x16_f16, f32 accumulate; "
                      "facet2vertex sums f32, its filter combination two fp16 pieces per operand" if args.f2f_half else
                      "f32 in HBM; facet2facet products and facet2vertex's filter combination on v_mfma_f32_32x32x16_f16 with "
                      "both operands split into two fp16 pieces (three piece products, about 22 significant bits), f32 "
                      "accumulate; the sums over points and facets in f32"),
               config=dict(workload=name + ("_f2f-half-products" if args.f2f_half and not bf16 else ""), facets=d["nf"], vertices=d["nv"], texture_points=d["T"], channels=C,
                           sh_degree=L, meshes=int(len(d["mf_in"])), algorithmic_bytes=total_bytes))
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline_conv(d, kind, torch)
    return res


def cpu_baseline_conv(d, kind, torch, budget_s=12.0):
    """Vectorised oracle (float32) on the host cores, mesh after mesh of the batch until `budget_s` is spent."""
    from oracle import torch_ref as R
    torch.set_num_threads(os.cpu_count() or 1)
    w_f2f, w_f2v, w_v2f = (torch.from_numpy(d[k]) for k in ("w_f2f", "w_f2v", "w_v2f"))
    f_off = np.concatenate([[0], np.cumsum(d["mf_in"])]).astype(np.int64)
    v_off = np.concatenate([[0], np.cumsum(d["nv_in"])]).astype(np.int64)
    t_off = np.concatenate([[0], np.cumsum(d["counts"])]).astype(np.int64)[f_off]
    done_f = done_t = n_mesh = 0
    spent = 0.0
    for m in range(len(d["mf_in"])):
        fa, fb, va, vb, ta, tb = f_off[m], f_off[m + 1], v_off[m], v_off[m + 1], t_off[m], t_off[m + 1]
        nf, nv = int(fb - fa), int(vb - va)
        f = torch.from_numpy(d["face"][fa:fb] - int(va))
        cum = torch.cumsum(torch.from_numpy(d["counts"][fa:fb]), 0, dtype=torch.int32)
        bary = torch.from_numpy(d["bary"][ta:tb])
        x = torch.from_numpy(d["x"][va:vb])
        own = torch.from_numpy(d["owner"][ta:tb] - int(fa))
        corner = f.long()[own]
        tex = x[corner[:, 0]] * bary[:, 0:1] + x[corner[:, 1]] * bary[:, 1:2] + x[corner[:, 2]] * bary[:, 2:3]
        tex = tex[:, :d["Cin"]].contiguous()
        sh, coeff = R.sph_harm(bary, d["L"]), R.sph_harm(torch.from_numpy(d["normal"][fa:fb]), d["L"])
        vt_map = torch.arange(nv, dtype=torch.int32)
        nfc = torch.from_numpy(d["nf_count"][va:vb].astype(np.int32))
        gy = torch.randn(nv, d["C"] * d["r"])
        t0 = time.perf_counter()
        if kind == "shapes":
            tex, sh = R.texture_fwd(x, f, bary, cum), R.sph_harm(bary, d["L"])
        y1 = R.f2f_fwd(tex, w_f2f, sh, cum)
        if kind == "shapes":
            y1 = y1 + R.v2f_fwd(x, w_v2f, f)
        R.f2v_fwd(y1, w_f2v, coeff, f, nfc, vt_map)
        g1, _ = R.f2v_bwd(gy, y1, w_f2v, coeff, f, nfc, vt_map)
        gt, _ = R.f2f_bwd(g1, tex, w_f2f, sh, cum)
        if kind == "shapes":
            R.texture_bwd(gt, nv, f, bary, cum)
            R.v2f_bwd(g1, x, w_v2f, f)
        spent += time.perf_counter() - t0
        done_f, done_t, n_mesh = done_f + nf, done_t + int(tb - ta), n_mesh + 1
        if spent >= budget_s:
            break
    return dict(value=done_f / spent / 1e6, unit="Mfacets/s", cores=torch.get_num_threads(), kind="port",
                sample="first %d of %d meshes of the batch (%d facets, %d texture points), one fwd+bwd pass each, %.1f s"
                       % (n_mesh, len(d["mf_in"]), done_f, done_t, spent))


def run_pool(args, torch):
    from picassoplus_amd import _lib, synthetic as S
    from picassoplus_amd.mesh.pi_modules import pool3d, unpool3d
    dev = torch.device("cuda:0")
    C, n = 128, 1024
    rng = np.random.default_rng(4000)
    nv = n * n
    vt_replace, vt_map, nvo = S.cluster_maps(rng, nv, mean=4.0, lo=1, hi=12, spatial=True)
    vr, vm = torch.from_numpy(vt_replace).to(dev), torch.from_numpy(vt_map).to(dev)
    x = torch.randn(nv, C, device=dev, requires_grad=True)
    vt_out = torch.zeros(nvo, 3, device=dev)
    g_c, g_f = torch.randn(nvo, C, device=dev), torch.randn(nv, C, device=dev)

    def step():
        y = pool3d.maxPool(x, vr, vm, vt_out)
        torch.autograd.grad(y, x, g_c)
        y = pool3d.avgPool(x, vr, vm, vt_out)
        torch.autograd.grad(y, x, g_c)
        c = y.detach().requires_grad_(True)
        u = unpool3d.interpolate(c, vr, vm)
        torch.autograd.grad(u, c, g_f)

    timer = EventTimer(torch)
    _lib.set_call_hook(timer)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer.on = True
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    _lib.set_call_hook(None)
    per_op = timer.summary()
    nb = {"pool_max_fwd": 4 * nv * C + 8 * nv + 8 * nvo * C, "pool_max_bwd": 8 * nvo * C + 4 * nv * C,
          "pool_avg_fwd": 4 * nv * C + 8 * nv + 4 * nvo * C, "pool_avg_bwd": 4 * nv * C + 8 * nv + 4 * nvo * C,
          "unpool_fwd": 4 * nvo * C + 8 * nv + 4 * nv * C, "unpool_bwd": 4 * nvo * C + 8 * nv + 4 * nv * C}
    dom = max(nb, key=lambda k: per_op[k])
    ach = nb[dom] / (per_op[dom] * 1e-3) / 1e9
    total = sum(nb.values())
    extra = {}
    if not args.no_cpu_baseline:
        # the oracle's restatement (float32 PyTorch-CPU scatter / gather ops) of the same six ops, once
        from oracle import torch_ref as R
        torch.set_num_threads(os.cpu_count() or 1)
        xc, rc, mc, gc, gf = x.detach().cpu(), vr.cpu(), vm.cpu(), g_c.cpu(), g_f.cpu()
        t0 = time.perf_counter()
        _, idx = R.maxpool_fwd(xc, rc, mc, nvo)
        R.maxpool_bwd(gc, nv, idx)
        ya = R.avgpool_fwd(xc, rc, mc, nvo)
        R.avgpool_bwd(gc, rc, mc)
        R.unpool_fwd(ya, rc, mc)
        R.unpool_bwd(gf, nvo, rc, mc)
        spent = time.perf_counter() - t0
        extra["cpu_baseline"] = dict(value=nv / spent / 1e6, unit="Mvertices/s", cores=torch.get_num_threads(), kind="port",
                                     sample="the whole grid (%d vertices, %d channels), one pass of the six ops, %.1f s" % (nv, C, spent))
    return dict(value=nv / (ms * 1e-3) / 1e6, unit="Mvertices/s", ms_per_step=ms, **extra,
                roofline=dict(bound="hbm", achieved=ach, peak=HBM_PEAK_GBS, unit="GB/s", frac=ach / HBM_PEAK_GBS,
                              traffic=measured_traffic("pool", "", dom), kernel=dom, kernel_ms=per_op[dom]),
                ops={k: dict(ms=per_op[k], gbps=nb[k] / (per_op[k] * 1e-3) / 1e9) for k in nb},
                hbm_gbps=total / (ms * 1e-3) / 1e9, hbm_frac=total / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                config=dict(workload="plane1024_pool_max+avg+unpool_C128_fp32_fwd+bwd", vertices=nv, coarse=nvo, channels=C))


def run_tail(args, torch):
    """The pointwise tail of a convolution on the scene batch's facet rows: act(rows @ W + b), 64 -> 64 channels,
    forward and backward (input, weight and bias gradients)."""
    from picassoplus_amd import _lib
    from picassoplus_amd.mesh.pi_modules import dense
    dev = torch.device("cuda:0")
    N, Ci, Co = int(2_400_000 * args.scale), 64, 64
    gen = torch.Generator(device=dev).manual_seed(5000)
    x = torch.randn(N, Ci, device=dev, generator=gen).requires_grad_(True)
    w = (torch.randn(Ci, Co, device=dev, generator=gen) / 8).requires_grad_(True)
    b = torch.randn(Co, device=dev, generator=gen).requires_grad_(True)
    g = torch.randn(N, Co, device=dev, generator=gen)

    def step():
        y = dense.dense_tail(x, w, b, True)
        return torch.autograd.grad(y, [x, w, b], g)

    timer = EventTimer(torch)
    _lib.set_call_hook(timer)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer.on = True
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    _lib.set_call_hook(None)
    per_op = timer.summary()
    # every operand once: the ReLU mask travels as one bit per entry (N * Co / 8 bytes) from the forward to the backward
    nb = {"dense_fwd": 4 * N * (Ci + Co) + N * Co // 8, "dense_bwd": 4 * N * (Co + Ci) + N * Co // 8 + 4 * N * Ci}
    fl = {"dense_fwd": 2.0 * N * Ci * Co, "dense_bwd": 4.0 * N * Ci * Co}
    dom = max(nb, key=lambda k: per_op[k])
    ach = nb[dom] / (per_op[dom] * 1e-3) / 1e9
    total = sum(nb.values())
    extra = {}
    if not args.no_cpu_baseline:
        # the oracle's restatement (float32 PyTorch-CPU ops) on slices of the same rows until about 10 s are spent
        from oracle import torch_ref as R
        torch.set_num_threads(os.cpu_count() or 1)
        xc, wc, bc, gc = x.detach().cpu(), w.detach().cpu(), b.detach().cpu(), g.cpu()
        rows = spent = 0
        chunk = 200_000
        while spent < 10.0 and rows + chunk <= N:
            xs, gs = xc[rows:rows + chunk], gc[rows:rows + chunk]
            t0 = time.perf_counter()
            R.dense_tail_bwd(gs, xs, wc, R.dense_tail_fwd(xs, wc, bc, True))
            spent += time.perf_counter() - t0
            rows += chunk
        extra["cpu_baseline"] = dict(value=rows / spent / 1e6, unit="Mrows/s", cores=torch.get_num_threads(), kind="port",
                                     sample="first %d of %d rows, one fwd+bwd pass, %.1f s" % (rows, N, spent))
    return dict(value=N / (ms * 1e-3) / 1e6, unit="Mrows/s", ms_per_step=ms, **extra,
                dtype="f32 in HBM; products on v_mfma_f32_32x32x16_bf16 with both operands split exactly into three bf16 "
                      "pieces (six piece products), f32 accumulate",
                roofline=dict(bound="hbm", achieved=ach, peak=HBM_PEAK_GBS, unit="GB/s", frac=ach / HBM_PEAK_GBS,
                              traffic=measured_traffic("tail", "", dom) if args.scale == 1.0 else None, kernel=dom,
                              kernel_ms=per_op[dom]),
                ops={k: dict(ms=per_op[k], gbps=nb[k] / (per_op[k] * 1e-3) / 1e9,
                             tflops=fl[k] / (per_op[k] * 1e-3) / 1e12) for k in nb},
                hbm_gbps=total / (ms * 1e-3) / 1e9, hbm_frac=total / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                config=dict(workload="scene_rows_dense_tail_64to64_relu_fp32_fwd+bwd", rows=N, in_channels=Ci,
                            out_channels=Co))


def run_f2vtail(args, torch):
    """The forward of an F2VConv3d module on the scene batch (64 channels, degree 3, 64 outputs, ReLU): the
    convolution and its pointwise tail as the two native passes (facet2vertex, then the product) and as the one pass
    that multiplies the vertex rows before they leave the chip, each without and with what a backward pass needs
    kept (the convolution's rows and the ReLU mask bits)."""
    from picassoplus_amd import _lib, synthetic as S
    from picassoplus_amd.mesh.pi_modules import dense, mesh_conv3d
    dev = torch.device("cuda:0")
    C, Co = 64, 64
    d = build_conv_inputs(S.scene_workload(scale=args.scale), C, 3, 3100, tex_counts=1)
    rng = np.random.default_rng(3101)
    T = lambda a, dt=None: torch.from_numpy(np.ascontiguousarray(a)).to(dev if dt is None else dev, dtype=dt)
    face, nfc, vmap = T(d["face"], torch.int32), T(d["nf_count"], torch.int32), T(d["vt_map"], torch.int32)
    xf = T(rng.uniform(-1, 1, (d["nf"], C)).astype(np.float32))
    coeff = T(rng.normal(0, 0.5, (d["nf"], 16)).astype(np.float32))
    filt = T(d["w_f2v"])
    w = T((rng.normal(0, 1, (C, Co)) / 8).astype(np.float32))
    b = T(rng.normal(0, 0.3, Co).astype(np.float32))
    variants = {
        "two_passes": lambda: dense.dense_tail_forward(mesh_conv3d.facet2vertex_forward(xf, filt, coeff, face, nfc, vmap), w, b, True),
        "one_pass": lambda: dense.f2v_dense_forward(xf, filt, coeff, face, nfc, vmap, w, b, True),
        "two_passes_kept": lambda: dense.dense_tail_forward(mesh_conv3d.facet2vertex_forward(xf, filt, coeff, face, nfc, vmap), w, b, True, with_bits=True),
        "one_pass_kept": lambda: dense.f2v_dense_forward(xf, filt, coeff, face, nfc, vmap, w, b, True, with_bits=True, keep_rows=True),
    }
    res, ops = {}, {}
    for name, fn in variants.items():
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        timer = EventTimer(torch)
        timer.on = True
        _lib.set_call_hook(timer)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        _lib.set_call_hook(None)
        res[name] = e0.elapsed_time(e1) / args.steps
        ops[name] = {k: round(v, 4) for k, v in timer.summary().items() if k.startswith(("f2v", "dense"))}
    Nv, Nf = d["nv"], d["nf"]
    # one pass, nothing kept: facet rows, coefficients, adjacency in; the module's output rows out
    nb = 4 * Nf * C + 4 * Nf * 16 + 12 * Nf + 8 * Nv + 4 * Nv * Co
    ms = res["one_pass"]
    ach = nb / (ms * 1e-3) / 1e9
    return dict(value=Nv / (ms * 1e-3) / 1e6, unit="Mvertices/s", ms_per_step=ms, variants_ms={k: round(v, 4) for k, v in res.items()},
                native_calls_ms=ops,
                dtype="f32 in HBM; both products on the fp16 matrix instructions with operands split into two fp16 pieces "
                      "(three piece products), f32 accumulate",
                roofline=dict(bound="hbm", achieved=ach, peak=HBM_PEAK_GBS, unit="GB/s", frac=ach / HBM_PEAK_GBS, traffic=None,
                              kernel="f2v_dense_fwd", kernel_ms=ops["one_pass"].get("f2v_dense_fwd", ms)),
                config=dict(workload="scene8x300k_F2VConv3d_forward_C64_L3_64out_relu_fp32", facets=Nf, vertices=Nv,
                            channels=C, out_channels=Co, algorithmic_bytes=nb))


def run_texture(args, torch):
    """Texture points of the scene batch's facets interpolated from 64-channel vertex features, with the SH basis of
    their barycentric coordinates (forward), and the transposed gather (backward)."""
    from picassoplus_amd import _lib, synthetic as S
    from picassoplus_amd.mesh.pi_modules import texture
    dev = torch.device("cuda:0")
    C, L = 64, 3
    mesh = S.scene_workload(seed=3000, n_rooms=8, scale=args.scale)
    d = build_conv_inputs(mesh, C, L, seed=3000)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    face, bary, x = t(d["face"]), t(d["bary"]), t(d["x"]).requires_grad_(True)
    cum = torch.cumsum(t(d["counts"]), 0, dtype=torch.int32)
    g = torch.randn(d["T"], C, device=dev, generator=torch.Generator(device=dev).manual_seed(1))

    def step():
        tex, _ = texture.interpolate(x, face, bary, cum, L)
        return torch.autograd.grad(tex, x, g)

    timer = EventTimer(torch)
    _lib.set_call_hook(timer)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer.on = True
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    _lib.set_call_hook(None)
    per_op = timer.summary()
    ops = ["texture_fwd", "texture_bwd"]
    bf = conv_bytes_flops(d, ops)
    dom = max(ops, key=lambda k: per_op[k])
    ach = bf[dom][0] / (per_op[dom] * 1e-3) / 1e9
    total = sum(b for b, _ in bf.values())
    extra = {}
    if not args.no_cpu_baseline:
        from oracle import torch_ref as R
        torch.set_num_threads(os.cpu_count() or 1)
        nf, nv = int(d["mf_in"][0]), int(d["nv_in"][0])               # first mesh of the batch
        nt = int(d["counts"][:nf].sum())
        f0, c0 = torch.from_numpy(d["face"][:nf]), torch.cumsum(torch.from_numpy(d["counts"][:nf]), 0, dtype=torch.int32)
        b0, x0, g0 = torch.from_numpy(d["bary"][:nt]), torch.from_numpy(d["x"][:nv]), torch.randn(nt, C)
        t0 = time.perf_counter()
        R.texture_fwd(x0, f0, b0, c0); R.sph_harm(b0, L); R.texture_bwd(g0, nv, f0, b0, c0)
        spent = time.perf_counter() - t0
        extra["cpu_baseline"] = dict(value=nf / spent / 1e6, unit="Mfacets/s", cores=torch.get_num_threads(), kind="port",
                                     sample="first of %d meshes (%d facets, %d texture points), one fwd+bwd pass, %.1f s"
                                            % (len(d["mf_in"]), nf, nt, spent))
    return dict(value=d["nf"] / (ms * 1e-3) / 1e6, ms_per_step=ms, **extra,
                roofline=dict(bound="hbm", achieved=ach, peak=HBM_PEAK_GBS, unit="GB/s", frac=ach / HBM_PEAK_GBS,
                              traffic=measured_traffic("texture", "", dom) if args.scale == 1.0 else None, kernel=dom,
                              kernel_ms=per_op[dom]),
                ops={k: dict(ms=per_op[k], gbps=bf[k][0] / (per_op[k] * 1e-3) / 1e9) for k in ops},
                hbm_gbps=total / (ms * 1e-3) / 1e9, hbm_frac=total / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                config=dict(workload="scene8x300k_texture_interpolation+SH_C64_L3_fp32_fwd+bwd", facets=d["nf"],
                            vertices=d["nv"], texture_points=d["T"], channels=C, sh_degree=L))


def run_pcloud(args, torch):
    """The point-cloud branch of a dual block on a coarse level of the scene batch (picasso/networks/pi2_blocks.py:43-62):
    every 16th vertex of the eight rooms, 128 channels, spherical-harmonic graph of the set on itself (range search,
    at most 16 neighbours, 17 weighted bins per pair), fuzzy depthwise convolution forward and backward.  The graph
    build (search + coefficients) is set-up, as in the reference's data pipeline, and reported beside the step."""
    from picassoplus_amd import _lib, synthetic as S
    from picassoplus_amd.point import utils as PU
    from picassoplus_amd.point.pi_modules import conv3d as pconv
    dev = torch.device("cuda:0")
    C, L, limit = 128, 3, 16
    mesh = S.scene_workload(seed=3000, n_rooms=8, scale=args.scale)
    nv_in = np.asarray(mesh["nv_in"], np.int64)
    start = np.concatenate([[0], np.cumsum(nv_in)])
    keep = np.concatenate([np.arange(start[b], start[b + 1], 16) for b in range(len(nv_in))])
    nv = np.array([len(np.arange(start[b], start[b + 1], 16)) for b in range(len(nv_in))], np.int32)
    xyz = torch.from_numpy(np.ascontiguousarray(mesh["vertex"][keep], dtype=np.float32)).to(dev)
    NV = torch.from_numpy(nv).to(dev)
    # radius: about 12 neighbours per point on the rooms' surfaces (points per area x pi r^2)
    v0 = mesh["vertex"][keep[:nv[0]]]                             # (the first room: its points lie on the faces of a box)
    ext = v0.max(0) - v0.min(0)
    radius = float(np.sqrt(12.0 / np.pi / (len(v0) / max(2.0 * (ext[0] * ext[1] + ext[1] * ext[2] + ext[0] * ext[2]), 1e-9))))
    # the graph build (range search + kernel bins): the first call carries one-time costs, the median of five more is
    # what a data pipeline pays per batch
    graph_times = []
    for _ in range(6):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        nn_cnt, nn_idx, nn_dst, filt_idx, filt_coeff = PU.build_sphere_harmonics(xyz, xyz, NV, NV, radius, L=L, nn_uplimit=limit)
        torch.cuda.synchronize()
        graph_times.append((time.perf_counter() - t0) * 1e3)
    graph_cold_ms, graph_ms = graph_times[0], float(np.median(graph_times[1:]))
    Np, P, T = xyz.shape[0], nn_idx.shape[0], filt_idx.shape[1]
    gen = torch.Generator(device=dev).manual_seed(6000)
    x = torch.randn(Np, C, device=dev, generator=gen).requires_grad_(True)
    w = (torch.randn(T, C, 1, device=dev, generator=gen) / 4).requires_grad_(True)
    g = torch.randn(Np, C, device=dev, generator=gen)

    def step():
        y = pconv.fuzzyconv3d(x, w, nn_cnt, nn_idx, filt_idx, filt_coeff)
        return torch.autograd.grad(y, [x, w], g)

    timer = EventTimer(torch)
    _lib.set_call_hook(timer)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer.on = True
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    _lib.set_call_hook(None)
    per_op = timer.summary()
    extra = {}
    # the other ops of a point level, once each beside the step (wall clock around synchronised calls, median of five):
    # sampling a quarter of every sample, the pooling graph of the sampled points, pooling and interpolation back
    from picassoplus_amd.point.pi_modules import nnquery as pnn, pool3d as ppool, sample as psample, unpool3d as punpool

    def wall(fn, reps=5):
        fn()
        ts = []
        for _ in range(reps):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            out = fn()
            torch.cuda.synchronize()
            ts.append((time.perf_counter() - t0) * 1e3)
        return float(np.median(ts)), out

    NQ = torch.from_numpy((nv // 4).astype(np.int32)).to(dev)
    other = {}
    other["fps_quarter"], picked = wall(lambda: psample.fps_(xyz, NV, NQ))
    q = xyz[picked.long()].contiguous()
    other["range_search_pool_graph"], (_, pcnt, pidx, _) = wall(lambda: pnn.range_search_(xyz, q, NV, NQ, radius=2 * radius, nnsample=32))
    gq = torch.randn(q.shape[0], C, device=dev, generator=gen)

    def fwd_bwd(fn, *a):
        def run():
            return torch.autograd.grad(fn(*a), [a[0]], gq if a[0] is x else g)
        return run

    other["max_pool_fwd_bwd"], _ = wall(fwd_bwd(ppool.maxPool, x, pcnt, pidx))
    other["avg_pool_fwd_bwd"], _ = wall(fwd_bwd(ppool.avgPool, x, pcnt, pidx))
    other["knn3_search"], (nn3, d3) = wall(lambda: pnn.knn3_search_(q, xyz, NQ, NV))
    xq = torch.randn(q.shape[0], C, device=dev, generator=gen).requires_grad_(True)
    other["interpolate_fwd_bwd"], _ = wall(fwd_bwd(punpool.interpolate, xq, PU.compute_unpool_weight(d3), nn3))
    extra["other_ops_ms"] = {k: round(v, 4) for k, v in other.items()}
    extra["other_ops_config"] = dict(sampled_points=int(q.shape[0]), pool_pairs=int(pidx.shape[0]))
    # every operand once: per pair its index pair, T bins and T weights, one gathered row of C floats; per point a row
    pair = 8 + 8 * T
    nb = {"point_conv_fwd": P * (pair + 4 * C) + 4 * Np * C + 4 * Np,
          "point_conv_bwd": P * (pair + 4 * C) + 4 * Np * C * 2 + 4 * Np}     # input and filter gradient from one walk over the pairs
    fl = {"point_conv_fwd": 2.0 * P * C * (T + 1), "point_conv_bwd": 2.0 * P * C * (2 * T + 2)}
    dom = max(nb, key=lambda k: per_op[k])
    ach = nb[dom] / (per_op[dom] * 1e-3) / 1e9
    total = sum(nb.values())
    if not args.no_cpu_baseline:
        # the oracle (numpy, float64) on the first sample's points and pairs
        from oracle import point_ref as R
        n0 = int(nv[0])
        cnt = nn_cnt[:n0].cpu().numpy()
        p0 = int(cnt.sum())
        idx, fi, fc = nn_idx[:p0].cpu().numpy(), filt_idx[:p0].cpu().numpy(), filt_coeff[:p0].cpu().numpy().astype(np.float64)
        xs, ws, gs = x[:n0].detach().cpu().numpy().astype(np.float64), w.detach().cpu().numpy().astype(np.float64), g[:n0].cpu().numpy().astype(np.float64)
        t0 = time.perf_counter()
        R.conv_fwd(xs, ws, cnt, idx, fi, fc)
        R.conv_bwd(gs, xs, ws, cnt, idx, fi, fc)
        spent = time.perf_counter() - t0
        extra["cpu_baseline"] = dict(value=n0 / spent / 1e6, unit="Mpoints/s", cores=1, kind="port",
                                     sample="first sample (%d points, %d pairs), one fwd+bwd pass, %.1f s" % (n0, p0, spent))
    return dict(value=Np / (ms * 1e-3) / 1e6, unit="Mpoints/s", ms_per_step=ms, graph_build_ms=graph_ms, graph_build_first_ms=graph_cold_ms, **extra, dtype="f32",
                roofline=dict(bound="hbm", achieved=ach, peak=HBM_PEAK_GBS, unit="GB/s", frac=ach / HBM_PEAK_GBS,
                              traffic=measured_traffic("pcloud", "", dom) if args.scale == 1.0 else None, kernel=dom,
                              kernel_ms=per_op[dom]),
                ops={k: dict(ms=per_op[k], gbps=nb[k] / (per_op[k] * 1e-3) / 1e9, tflops=fl[k] / (per_op[k] * 1e-3) / 1e12)
                     for k in nb},
                hbm_gbps=total / (ms * 1e-3) / 1e9, hbm_frac=total / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                config=dict(workload="scene8_every16th_vertex_fuzzy_pointconv_C128_L3_nn16_fp32_fwd+bwd", points=Np, pairs=P,
                            bins_per_pair=T, channels=C, radius=radius, meshes=int(len(nv))))


def run_decimate(args, torch):
    """Mesh decimation of the scene batch to a quarter of its vertices (picasso/mesh/pi_modules/decimate.py:5-52): the
    producer of the cluster maps the pooling ops take.  One step = the whole loop of simplification rounds; the
    native calls (quadrics, edge costs, host clustering, cluster composition, position averaging) are timed per entry
    point, the rest of a step is the integer sorts / scans / compactions between them (PyTorch ops)."""
    from picassoplus_amd import _lib, synthetic as S
    from picassoplus_amd.mesh.pi_modules import decimate as D
    dev = torch.device("cuda:0")
    mesh = S.scene_workload(seed=3000, n_rooms=8, scale=args.scale)
    t = lambda a, dt: torch.from_numpy(np.ascontiguousarray(a)).to(dt).to(dev)
    vertex, face = t(mesh["vertex"], torch.float32), t(mesh["face"], torch.int32)
    nv_in, mf_in = t(mesh["nv_in"], torch.int32), t(mesh["mf_in"], torch.int32)
    nv_out = (nv_in // 4).to(torch.int32)
    geometry = D.compute_triangle_geometry_(vertex, face)
    Nv, Nf = vertex.shape[0], face.shape[0]
    rounds = []

    def step():
        out = D.mesh_decimation_(vertex, face, geometry, nv_in, mf_in, nv_out)
        return out

    timer = EventTimer(torch)
    _lib.set_call_hook(timer)
    for _ in range(max(1, min(args.warmup, 2))):
        out = step()
    torch.cuda.synchronize()
    timer.on = True
    steps = max(1, min(args.steps, 5))
    t0 = time.perf_counter()
    for _ in range(steps):
        out = step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    _lib.set_call_hook(None)
    per_step = timer.totals(steps)
    per_call = timer.summary()
    calls = {}
    for name, _, _ in timer.pairs:
        k = name.replace("pmesh_", "")
        calls[k] = calls.get(k, 0) + 1
    n_rounds = calls.get("edge_costs", steps) // steps
    # the edge-cost kernel on the first round's candidate edges: per edge two quadrics (10 floats each), two positions,
    # two indices in, one cost out
    dom = "edge_costs"
    quadric, evi, evj = D.vertex_quadrics(vertex, face, geometry)
    D.edge_costs(vertex, quadric, evi, evj)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        D.edge_costs(vertex, quadric, evi, evj)
    e1.record()
    torch.cuda.synchronize()
    edge_ms = e0.elapsed_time(e1) / 5
    n_edges0 = int(evi.shape[0])
    edge_bytes = n_edges0 * (2 * 40 + 2 * 4 * vertex.shape[1] + 8 + 4)
    ach = edge_bytes / (edge_ms * 1e-3) / 1e9
    extra = {}
    if not args.no_cpu_baseline:
        from oracle import decimate_ref as R
        # the numpy oracle on the first sample, one round
        n0, m0 = int(mesh["nv_in"][0]), int(mesh["mf_in"][0])
        v0 = np.ascontiguousarray(mesh["vertex"][:n0], dtype=np.float32)
        f0 = np.ascontiguousarray(mesh["face"][:m0], dtype=np.int32)
        t0 = time.perf_counter()
        R.simplify(v0, f0, R.triangle_geometry(v0, f0), np.array([n0]), np.array([m0]), np.array([n0 - n0 // 4]))
        spent = time.perf_counter() - t0
        extra["cpu_baseline"] = dict(value=n0 / spent / 1e6, unit="Mvertices/s", cores=1, kind="port",
                                     sample="first sample (%d vertices, %d facets), ONE simplification round, %.1f s" % (n0, m0, spent))
    native = sum(per_step.values())
    return dict(value=Nv / (ms * 1e-3) / 1e6, unit="Mvertices/s", ms_per_step=ms, steps_timed=steps, rounds=n_rounds, **extra,
                dtype="f32 (quadrics, costs), int32 (maps)",
                roofline=dict(bound="hbm", achieved=ach, peak=HBM_PEAK_GBS, unit="GB/s", frac=ach / HBM_PEAK_GBS, traffic=None,
                              kernel=dom + " (first round, %d candidate edges)" % n_edges0, kernel_ms=edge_ms),
                native_ms_per_step=native, ops_ms_per_step=per_step, ops_ms_per_call=per_call,
                vertices_out=int(out[0].shape[0]), facets_out=int(out[1].shape[0]),
                config=dict(workload="scene8x300k_decimation_to_quarter_fp32", vertices=Nv, facets=Nf, meshes=int(len(mesh["nv_in"]))))


def run_hierarchy(args, torch):
    """Encoder-decoder stack of the mesh modules over one 2 M-facet mesh and four 4:1 coarser levels: per level
    V2F + (texture interpolation -> F2F) -> F2V at widths 32/64/128/256, max / avg pooling between levels, then
    unpooling back to the finest level with a pointwise layer per level; forward + backward.  Also times every
    level's block alone, to show how the kernels' shares move with mesh size and width."""
    from torch import nn
    from picassoplus_amd import _lib, synthetic as S
    from picassoplus_amd.mesh import layers
    from picassoplus_amd.mesh.pi_modules import texture
    dev = torch.device("cuda:0")
    L, NL = 3, 4
    W = [32, 64, 128, 256, 256]
    cells = 1024 if args.scale == 1.0 else max(16, int(1024 * args.scale ** 0.5) // 16 * 16)
    meshes = S.hierarchy_workload(seed=5000, cells=cells, levels=NL)
    rng = np.random.default_rng(5000)
    torch.manual_seed(5000)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    lv = []
    for l in range(NL):
        m = meshes[l]
        v, f = m["vertex"], m["face"]
        nv, nf = v.shape[0], f.shape[0]
        normal, _ = S.triangle_normals_areas(v, f)
        counts, bary, _ = S.texture_points(rng, nf, rng.integers(1, 4, nf).astype(np.int32))
        lv.append(dict(nv=nv, nf=nf, T=int(counts.sum()), C=W[l], Cin=W[l], r=1, B=(L + 1) ** 2, face=t(f),
                       nfc=t(np.maximum(S.vertex_facet_count(f, np.arange(nv), nv), 1).astype(np.int32)),
                       ident=torch.arange(nv, dtype=torch.int32, device=dev),
                       coeff=layers.sph_harm_values(t(normal.astype(np.float32)), L), counts=t(counts),
                       cum=torch.cumsum(t(counts), 0, dtype=torch.int32), bary=t(bary.astype(np.float32)),
                       vr=t(m["vt_replace"]), vm=t(m["vt_map"]), vt_out=torch.zeros(m["nv_out"], 3, device=dev),
                       np_face=f, np_counts=counts, np_bary=bary, np_normal=normal,
                       v2f=layers.V2FConv3d(W[l], W[l], L, with_bn=False).to(dev),
                       f2f=layers.F2FConv3d(W[l], W[l], L, with_bn=False).to(dev),
                       f2v=layers.F2VConv3d(W[l], W[l + 1], L, with_bn=False).to(dev),
                       pool=layers.Pool3d("max" if l % 2 == 0 else "avg"),
                       up=layers.PerItemConv3d(W[l + 1], W[l], with_bn=False).to(dev)))
    params = [p for d in lv for k in ("v2f", "f2f", "f2v", "up") for p in d[k].parameters()]
    x0 = torch.randn(lv[0]["nv"], W[0], device=dev, requires_grad=True)
    gy = torch.randn(lv[0]["nv"], W[0], device=dev)

    def block(d, x):
        tex, sh = texture.interpolate(x, d["face"], d["bary"], d["cum"], L)
        y = d["v2f"](x, d["face"]) + d["f2f"](tex, sh, d["counts"])
        z = d["f2v"](y, d["face"], d["nfc"], d["ident"], d["coeff"])
        return z, d["pool"](z, d["vr"], d["vm"], d["vt_out"])

    def step():
        x, skips = x0, []
        for d in lv:
            z, x = block(d, x)
            skips.append(z)
        for d, z in zip(reversed(lv), reversed(skips)):
            x = d["up"](z + layers.Unpool3d.forward(x, d["vr"], d["vm"]))
        return torch.autograd.grad(x, [x0] + params, gy)

    def timed(fn):
        # the step's time from a plain loop, the per-op times from a second loop with an event pair around every native
        # call (some 150 calls per step here: the event records alone add 4 % to a full-size step and a third to a small one)
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
        timer = EventTimer(torch)
        _lib.set_call_hook(timer)
        timer.on = True
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        _lib.set_call_hook(None)
        return ms, timer.totals(args.steps)

    ms, per_op = timed(step)
    graph_ms = None
    if args.graph:
        # the same step recorded once and replayed: what the launches of about 150 kernels per step cost on the host
        # side no longer lies between the kernels (matters for small meshes; a 2 M-facet step is bound by the GPU)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            recorded = step()
        for _ in range(args.warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        eager = step()
        torch.cuda.synchronize()
        if not all(torch.equal(a, b) for a, b in zip(recorded, eager)):
            sys.exit("bench.py --graph: the replayed step differs from the eager one")
    # every level's block alone (forward + backward of its five ops and their tails)
    conv_ops = ["v2f_fwd", "texture_fwd", "f2f_fwd", "f2v_fwd", "f2v_bwd", "f2f_bwd_texture", "f2f_bwd_filter",
                "texture_bwd", "v2f_bwd"]
    report, best = [], None
    for l, d in enumerate(lv):
        xin = torch.randn(d["nv"], W[l], device=dev, requires_grad=True)
        gz, gp = torch.randn(d["nv"], W[l + 1], device=dev), torch.randn(d["vt_out"].shape[0], W[l + 1], device=dev)
        own = [p for k in ("v2f", "f2f", "f2v") for p in d[k].parameters()]

        def one(d=d, xin=xin, gz=gz, gp=gp, own=own):
            z, p = block(d, xin)
            return torch.autograd.grad([z, p], [xin] + own, [gz, gp])

        lms, lops = timed(one)
        bf = conv_bytes_flops(d, conv_ops)
        report.append(dict(level=l, facets=d["nf"], vertices=d["nv"], texture_points=d["T"], channels=W[l], ms=lms,
                           ops_ms={k: round(v, 4) for k, v in sorted(lops.items())},
                           share={k: round(v / sum(lops.values()), 3) for k, v in sorted(lops.items())}))
        for k in conv_ops:
            if k in lops and (best is None or lops[k] > best[0]):
                best = (lops[k], k, l, bf[k])
    dom_ms, dom, dl, (nbytes, nflops) = best
    if dom.startswith("f2f"):
        ach = nflops / (dom_ms * 1e-3) / 1e12
        roof = dict(bound="mfma", achieved=ach, peak=MFMA_F16_PEAK_TFLOPS / F2F_PIECE_PRODUCTS, unit="TFLOP/s",
                    peak_basis="fp16 dense MFMA 2500 TFLOP/s / 3 piece products per fp32-accurate product",
                    frac_of_fp32_mfma_peak=ach / MFMA_F32_PEAK_TFLOPS)
    else:
        roof = dict(bound="hbm", achieved=nbytes / (dom_ms * 1e-3) / 1e9, peak=HBM_PEAK_GBS, unit="GB/s")
    roof.update(frac=roof["achieved"] / roof["peak"], traffic=None, kernel="%s@level%d" % (dom, dl), kernel_ms=dom_ms)
    res = dict(value=lv[0]["nf"] / (ms * 1e-3) / 1e6, ms_per_step=ms, roofline=roof,
               dtype="f32 in HBM; facet2facet products two fp16 pieces per operand, pointwise tails three bf16 pieces per "
                     "operand, f32 accumulate; everything else f32",
               ops_ms_per_step={k: round(v, 4) for k, v in sorted(per_op.items())}, levels=report,
               config=dict(workload="grid%d_4levels_V2F+texture+F2F+F2V+pool+unpool_C32-256_L3_fp32_fwd+bwd" % cells,
                           facets=[d["nf"] for d in lv], vertices=[d["nv"] for d in lv] + [int(lv[-1]["vt_out"].shape[0])],
                           channels=W[:NL], sh_degree=L))
    if graph_ms is not None:
        res["graph_replay_ms_per_step"] = graph_ms
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline_block(lv[-1], W[NL - 1], L, torch)
    return res


def cpu_baseline_block(d, C, L, torch):
    """The oracle's restatement (float32 PyTorch-CPU ops) of the coarsest level's convolutions, forward + backward."""
    from oracle import torch_ref as R
    from picassoplus_amd import synthetic as S
    torch.set_num_threads(os.cpu_count() or 1)
    rng = np.random.default_rng(1)
    nv, nf, B = d["nv"], d["nf"], (L + 1) ** 2
    f = torch.from_numpy(d["np_face"])
    cum = torch.cumsum(torch.from_numpy(d["np_counts"]), 0, dtype=torch.int32)
    bary = torch.from_numpy(d["np_bary"].astype(np.float32))
    coeff = R.sph_harm(torch.from_numpy(d["np_normal"].astype(np.float32)), L)
    x, gy = torch.randn(nv, C), torch.randn(nv, C)
    w_v2f = torch.from_numpy(S.xavier_uniform(rng, (3, C, 1), C, 3 * C).astype(np.float32))
    w_f2f = torch.from_numpy(S.xavier_uniform(rng, (C, C, B), C * B, C * B).astype(np.float32))
    w_f2v = torch.from_numpy(S.xavier_uniform(rng, (B, C, 1), C, B * C).astype(np.float32))
    nfc, ident = d["nfc"].cpu(), torch.arange(nv, dtype=torch.int32)
    t0 = time.perf_counter()
    tex, sh = R.texture_fwd(x, f, bary, cum), R.sph_harm(bary, L)
    y = R.f2f_fwd(tex, w_f2f, sh, cum) + R.v2f_fwd(x, w_v2f, f)
    R.f2v_fwd(y, w_f2v, coeff, f, nfc, ident)
    g1, _ = R.f2v_bwd(gy, y, w_f2v, coeff, f, nfc, ident)
    gt, _ = R.f2f_bwd(g1, tex, w_f2f, sh, cum)
    R.texture_bwd(gt, nv, f, bary, cum)
    R.v2f_bwd(g1, x, w_v2f, f)
    spent = time.perf_counter() - t0
    return dict(value=nf / spent / 1e6, unit="Mfacets/s", cores=torch.get_num_threads(), kind="port",
                sample="convolutions of the coarsest conv level only (%d facets, %d channels; no tails, pools or "
                       "other levels), one fwd+bwd pass, %.1f s" % (nf, C, spent))


def main():
    args = parse()
    if args.traffic_from:
        write_traffic(args)
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: this path keeps whole meshes on one device and nothing here "
              "uses a second one; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    from picassoplus_amd import _lib
    _lib.load()
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (torch.cuda.is_available() is False)", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    if args.f2f_half:
        os.environ["PMESH_F2F_HALF"] = "1"
        _lib.reload_options()                       # the library reads its switches once
    if args.workload == "pool":
        res = run_pool(args, torch)
    elif args.workload == "tail":
        res = run_tail(args, torch)
    elif args.workload == "f2vtail":
        res = run_f2vtail(args, torch)
    elif args.workload == "hierarchy":
        res = run_hierarchy(args, torch)
    elif args.workload == "texture":
        res = run_texture(args, torch)
    elif args.workload == "pcloud":
        res = run_pcloud(args, torch)
    elif args.workload == "decimate":
        res = run_decimate(args, torch)
    else:
        res = run_conv_layer(args, torch, args.workload)
    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda:0").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    line = dict(metric="mesh-conv layer fwd+bwd throughput", value=res.pop("value"), unit=res.pop("unit", "Mfacets/s"),
                n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=res.pop("ms_per_step"),
                higher_is_better=True, scaling="weak", vs_baseline=None,
                dtype=res.pop("dtype", "f32"), data="synthetic", build_id=build_id())
    line.update(res)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
