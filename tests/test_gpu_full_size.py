"""GPU checks at the benchmark's full sizes through properties that do not need a full CPU oracle run:
adjoint identities (each op is linear in its features and in its filter), oracle parity on a random
sample of facets, invariance under the optional facet order, and the pooling invariants."""
import numpy as np
import pytest
import torch

from oracle import loops
from picassoplus_amd import _lib, synthetic as S
from picassoplus_amd.mesh import topology
from picassoplus_amd.mesh.layers import sph_harm_values
from picassoplus_amd.mesh.pi_modules import conv3d, mesh_conv3d, pool3d, texture, unpool3d
from util import assert_close, dev

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def _dot(a, b):
    return float((a.double() * b.double()).sum())


def _adjoint_ok(lhs, rhs, scale, what, tol=1e-5):
    assert abs(lhs - rhs) <= tol * scale, "%s: %.9g vs %.9g (scale %.3g)" % (what, lhs, rhs, scale)


@pytest.fixture(scope="module")
def scene(cuda):
    """The bench's scene batch: 8 rooms, about 2.4 M facets, area-scaled texture counts 1..9, C = 64."""
    say("building the scene workload")
    rng = np.random.default_rng(3000)
    mesh = S.scene_workload(seed=3000, n_rooms=8, scale=1.0)
    v, f = mesh["vertex"], mesh["face"]
    nv, nf = v.shape[0], f.shape[0]
    normal, area = S.triangle_normals_areas(v, f)
    counts, bary, owner = S.texture_points(rng, nf, S.area_scaled_texture_counts(area))
    C, L = 64, 3
    d = dict(nv=nv, nf=nf, T=int(counts.sum()), C=C, counts=counts)
    d["face"] = dev(f, cuda)
    d["cum"] = torch.cumsum(dev(counts, cuda), 0, dtype=torch.int32)
    d["bary"] = dev(bary.astype(np.float32), cuda)
    d["bary64"], d["face_np"] = bary, f
    d["sh"] = sph_harm_values(d["bary"], L)
    d["coeff"] = sph_harm_values(dev(normal.astype(np.float32), cuda), L)
    d["tex"] = dev(rng.uniform(-1, 1, (d["T"], C)).astype(np.float32), cuda)
    d["w_f2f"] = dev(S.xavier_uniform(rng, (C, C, 16), C * 16, C * 16).astype(np.float32), cuda)
    d["w_f2v"] = dev(S.xavier_uniform(rng, (16, C, 1), C, 16 * C).astype(np.float32), cuda)
    d["nfc"] = dev(np.maximum(S.vertex_facet_count(f, np.arange(nv), nv), 1).astype(np.int32), cuda)
    d["vt_map"] = dev(np.arange(nv, dtype=np.int32), cuda)
    return d


def test_f2f_full_size_adjoints_and_sample_parity(cuda, scene):
    d = scene
    say("case f2f full size", d["nf"], d["T"])
    gen = torch.Generator(device=cuda).manual_seed(5)
    g = torch.randn(d["nf"], d["C"], device=cuda, generator=gen)
    tex = d["tex"].clone().requires_grad_(True)
    w = d["w_f2f"].clone().requires_grad_(True)
    out = conv3d.facet2facet(tex, w, d["sh"], d["cum"])
    gtex, gw = torch.autograd.grad(out, [tex, w], g)
    torch.cuda.synchronize()
    lhs = _dot(out, g)
    scale = float(out.double().norm() * g.double().norm())
    _adjoint_ok(lhs, _dot(tex, gtex), scale, "<f2f(tex), g> = <tex, grad_texture>")
    _adjoint_ok(lhs, _dot(w, gw), scale, "<f2f(tex), g> = <W, grad_filter>")

    # oracle parity on a sample of facets: outputs and texture gradients of a facet depend on that facet only
    rng = np.random.default_rng(6)
    pick = np.sort(rng.choice(d["nf"], 1500, replace=False))
    counts = d["counts"]
    start = np.concatenate([[0], np.cumsum(counts)])[:-1]
    rows = np.concatenate([np.arange(start[f], start[f] + counts[f]) for f in pick]).astype(np.int64)
    rows_t = torch.from_numpy(rows).to(cuda)
    sub_tex = d["tex"][rows_t].cpu().numpy().astype(np.float64)
    sub_sh = d["sh"][rows_t].cpu().numpy().astype(np.float64)
    sub_cum = np.cumsum(counts[pick]).astype(np.int32)
    wt = d["w_f2f"].cpu().numpy().astype(np.float64)
    pick_t = torch.from_numpy(pick).to(cuda)
    sub_g = g[pick_t].cpu().numpy().astype(np.float64)
    ref_out = loops.f2f_fwd(sub_tex, wt, sub_sh, sub_cum)
    ref_gtex, _ = loops.f2f_bwd(sub_g, sub_tex, wt, sub_sh, sub_cum)
    assert_close(out.detach()[pick_t], ref_out, "f2f out (sampled facets)")
    assert_close(gtex[rows_t], ref_gtex, "f2f grad_texture (sampled facets)")

    # the filter gradient element by element, from the reference's point-wise form in float64 (blocks of points)
    say("  grad_filter against the float64 oracle")
    from oracle import torch_ref as R
    torch.set_num_threads(16)
    ref_gw = R.f2f_bwd_filter_pointwise(g.cpu().double(), d["tex"].cpu().double(), d["sh"].cpu().double(), d["cum"].cpu())
    assert_close(gw, ref_gw.numpy(), "f2f grad_filter (whole batch, element by element)")

    # the facet order is an optimisation only.  A facet's power-of-two operand scale can depend on its workgroup
    # (all of it falls back to exact row maxima when one facet exceeds its first bound), which moves results by
    # an ulp at most; with no such fallback, as on this data, nothing changes by a bit
    T, Cin = d["tex"].shape
    ws_n = _lib.query("pmesh_f2f_fwd_workspace_bytes", Cin, d["C"], 16)
    ws = torch.empty(ws_n, dtype=torch.uint8, device=cuda)
    out2 = torch.empty_like(out)
    _lib.call("pmesh_f2f_fwd", d["tex"].data_ptr(), d["w_f2f"].data_ptr(), d["sh"].data_ptr(), d["cum"].data_ptr(),
              None, out2.data_ptr(), ws.data_ptr(), ws_n, T, d["nf"], Cin, d["C"], 16,
              torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert float((out2 - out.detach()).abs().max()) <= 2e-7 * float(out.detach().abs().max())


def test_f2v_full_size_adjoints(cuda, scene):
    d = scene
    say("case f2v full size", d["nf"], d["nv"])
    gen = torch.Generator(device=cuda).manual_seed(7)
    x = torch.randn(d["nf"], d["C"], device=cuda, generator=gen).requires_grad_(True)
    w = d["w_f2v"].clone().requires_grad_(True)
    g = torch.randn(d["nv"], d["C"], device=cuda, generator=gen)
    out = conv3d.facet2vertex(x, w, d["coeff"], d["face"], d["nfc"], d["vt_map"])
    gx, gw = torch.autograd.grad(out, [x, w], g)
    torch.cuda.synchronize()
    lhs = _dot(out, g)
    scale = float(out.double().norm() * g.double().norm())
    _adjoint_ok(lhs, _dot(x, gx), scale, "<f2v(x), g> = <x, grad_input>")
    _adjoint_ok(lhs, _dot(w, gw), scale, "<f2v(x), g> = <filter, grad_filter>")
    # oracle parity: output rows of sampled vertices (a row depends on the facets around that vertex only),
    # grad_input rows of sampled facets (a row depends on the facet's three vertices only), and the whole
    # filter gradient element by element from the float64 restatement
    say("  f2v sampled rows and grad_filter against the float64 oracle")
    from oracle import torch_ref as R
    torch.set_num_threads(16)
    rng = np.random.default_rng(11)
    f_np = d["face_np"].astype(np.int64)
    nfc_np = d["nfc"].cpu().numpy()
    x_np, w_np = x.detach().cpu().numpy().astype(np.float64), w.detach().cpu().numpy().astype(np.float64)
    coeff_np = d["coeff"].cpu().numpy().astype(np.float64)
    pick_v = np.sort(rng.choice(d["nv"], 2000, replace=False))
    is_pick = np.zeros(d["nv"], bool)
    is_pick[pick_v] = True
    around = np.nonzero(is_pick[f_np].any(1))[0]                 # facets with a sampled corner
    sub_out = loops.f2v_fwd(x_np[around], w_np, coeff_np[around], f_np[around].astype(np.int32), nfc_np,
                            np.arange(d["nv"], dtype=np.int32))
    assert_close(out.detach()[torch.from_numpy(pick_v).to(cuda)], sub_out[pick_v], "f2v out (sampled vertices)")
    pick_f = np.sort(rng.choice(d["nf"], 2000, replace=False))
    sub_gin, _ = loops.f2v_bwd(g.cpu().numpy().astype(np.float64), x_np[pick_f], w_np, coeff_np[pick_f],
                               f_np[pick_f].astype(np.int32), nfc_np, np.arange(d["nv"], dtype=np.int32))
    assert_close(gx[torch.from_numpy(pick_f).to(cuda)], sub_gin, "f2v grad_input (sampled facets)")
    _, ref_gw = R.f2v_bwd(g.cpu().double(), x.detach().cpu().double(), w.detach().cpu().double(), d["coeff"].cpu().double(),
                          d["face"].cpu(), d["nfc"].cpu(), d["vt_map"].cpu())
    assert_close(gw, ref_gw.numpy(), "f2v grad_filter (whole batch, element by element)")
    del ref_gw

    # a constant field with unit coefficient 0 and all other coefficients zero is averaged to itself
    coeff = torch.zeros_like(d["coeff"])
    coeff[:, 0] = 1.0
    w1 = torch.zeros_like(d["w_f2v"])
    w1[0] = 1.0
    ones = torch.full((d["nf"], d["C"]), 0.75, device=cuda)
    y = mesh_conv3d.facet2vertex_forward(ones, w1, coeff, d["face"], d["nfc"], d["vt_map"])
    torch.cuda.synchronize()
    touched = torch.zeros(d["nv"], dtype=torch.bool, device=cuda)
    touched[d["face"].long().reshape(-1)] = True
    assert float((y[touched] - 0.75).abs().max()) <= 1e-6


def test_f2v_with_its_tail_full_size(cuda, scene):
    """facet2vertex and its pointwise tail in one pass on the whole scene batch: the kept rows are the convolution
    kernel's rows bit for bit, the output agrees with the two native passes (each of which is checked against the
    oracle at this size) and with the float64 oracle composition on sampled vertices, the mask bits with the output."""
    from oracle import torch_ref as R
    from picassoplus_amd.mesh.pi_modules import dense, mesh_conv3d
    d = scene
    say("case f2v + tail full size", d["nf"], d["nv"])
    gen = torch.Generator(device=cuda).manual_seed(17)
    C, Co = d["C"], 64
    x = torch.randn(d["nf"], C, device=cuda, generator=gen)
    w = torch.randn(C, Co, device=cuda, generator=gen) / 8
    b = torch.randn(Co, device=cuda, generator=gen)
    args = (x, d["w_f2v"], d["coeff"], d["face"], d["nfc"], d["vt_map"])
    assert dense.f2v_dense_supported(x, d["w_f2v"], d["coeff"], w)
    out, bits, rows = dense.f2v_dense_forward(*args, w, b, True, with_bits=True, keep_rows=True)
    conv = mesh_conv3d.facet2vertex_forward(*args)
    two = dense.dense_tail_forward(conv, w, b, True)
    torch.cuda.synchronize()
    assert torch.equal(rows, conv)
    assert float((out - two).abs().max()) <= 2e-6 * float(two.abs().max())
    assert torch.equal(dense.f2v_dense_forward(*args, w, b, True), out)
    cols = torch.arange(Co, device=cuda)
    assert torch.equal(((bits[:, cols // 32] >> (cols % 32)) & 1).bool(), out > 0)
    rng = np.random.default_rng(19)
    f_np = d["face_np"].astype(np.int64)
    pick_v = np.sort(rng.choice(d["nv"], 2000, replace=False))
    is_pick = np.zeros(d["nv"], bool)
    is_pick[pick_v] = True
    around = np.nonzero(is_pick[f_np].any(1))[0]
    sub = loops.f2v_fwd(x.cpu().numpy().astype(np.float64)[around], d["w_f2v"].cpu().numpy().astype(np.float64),
                        d["coeff"].cpu().numpy().astype(np.float64)[around], f_np[around].astype(np.int32),
                        d["nfc"].cpu().numpy(), np.arange(d["nv"], dtype=np.int32))
    ref = R.dense_tail_fwd(torch.from_numpy(sub[pick_v]), w.double().cpu(), b.double().cpu(), True).numpy()
    assert_close(out[torch.from_numpy(pick_v).to(cuda)], ref, "f2v + tail out (sampled vertices)")


def test_v2f_full_size_adjoints(cuda, scene):
    d = scene
    gen = torch.Generator(device=cuda).manual_seed(8)
    x = torch.randn(d["nv"], d["C"], device=cuda, generator=gen).requires_grad_(True)
    w = torch.randn(3, d["C"], 1, device=cuda, generator=gen).requires_grad_(True)
    g = torch.randn(d["nf"], d["C"], device=cuda, generator=gen)
    out = conv3d.vertex2facet(x, w, d["face"])
    gx, gw = torch.autograd.grad(out, [x, w], g)
    torch.cuda.synchronize()
    lhs = _dot(out, g)
    scale = float(out.double().norm() * g.double().norm())
    _adjoint_ok(lhs, _dot(x, gx), scale, "<v2f(x), g> = <x, grad_input>")
    _adjoint_ok(lhs, _dot(w, gw), scale, "<v2f(x), g> = <filter, grad_filter>")


def test_texture_interpolation_full_size(cuda, scene):
    """Adjoint identity, the invariants of barycentric weights (constants stay constant), the fused basis against the
    stand-alone kernel, and oracle parity on a random sample of facets."""
    d = scene
    say("case texture full size", d["nf"], d["T"])
    gen = torch.Generator(device=cuda).manual_seed(9)
    x = torch.randn(d["nv"], d["C"], device=cuda, generator=gen).requires_grad_(True)
    g = torch.randn(d["T"], d["C"], device=cuda, generator=gen)
    tex, sh = texture.interpolate(x, d["face"], d["bary"], d["cum"], 3)
    (gx,) = torch.autograd.grad(tex, x, g)
    torch.cuda.synchronize()
    assert torch.equal(sh, d["sh"])
    _adjoint_ok(_dot(tex, g), _dot(x, gx), float(tex.double().norm() * g.double().norm()), "<tex(x), g> = <x, grad_input>")
    const = texture.interpolate(torch.full((d["nv"], 8), 2.5, device=cuda), d["face"], d["bary"], d["cum"], None)
    assert float((const - 2.5).abs().max()) < 1e-5
    # every gradient row sums what its vertex's corners received: total mass is preserved (weights sum to one)
    _adjoint_ok(float(gx.double().sum()), float(g.double().sum()), float(g.double().abs().sum()), "sum of grad_input = sum of grad_texture")
    # oracle on 500 random facets: their rows of the output
    rng = np.random.default_rng(10)
    pick = np.sort(rng.choice(d["nf"], 500, replace=False))
    cum = np.cumsum(d["counts"])
    xs = x.detach().cpu().numpy().astype(np.float64)
    tex_np = tex.detach().cpu().numpy()
    for f in pick[:500]:
        k0, k1 = (cum[f - 1] if f else 0), cum[f]
        ref = d["bary64"][k0:k1] @ xs[d["face_np"][f].astype(np.int64)]
        assert np.abs(tex_np[k0:k1] - ref).max() <= 1e-5 * max(np.abs(ref).max(), 1.0)


def test_pool_full_size_invariants(cuda):
    """1024 x 1024 grid, about 261 k clusters of 1..12 vertices, C = 128."""
    say("case pool full size")
    nv, C = 1024 * 1024, 128
    rng = np.random.default_rng(4000)
    vt_replace, vt_map, nvo = S.cluster_maps(rng, nv, mean=4.0, lo=1, hi=12, spatial=True)
    vr, vm = dev(vt_replace, cuda), dev(vt_map, cuda)
    gen = torch.Generator(device=cuda).manual_seed(9)
    x = torch.randn(nv, C, device=cuda, generator=gen).requires_grad_(True)
    vt_out = torch.zeros(nvo, 3, device=cuda)
    g = torch.randn(nvo, C, device=cuda, generator=gen)
    # cluster id of every fine vertex, from the maps' definition
    rep = torch.where(vr < 0, -vr, torch.arange(nv, device=cuda, dtype=torch.int32)).long()
    cl = vm.long()[rep]
    assert int(cl.min()) >= 0 and int(cl.max()) == nvo - 1

    y = pool3d.maxPool(x, vr, vm, vt_out)
    (gx,) = torch.autograd.grad(y, x, g)
    ref = torch.full((nvo, C), -float("inf"), device=cuda).scatter_reduce(0, cl[:, None].expand(-1, C), x.detach(), "amax")
    assert torch.equal(y.detach(), ref)                                     # max values are exact
    assert abs(_dot(gx, torch.ones_like(gx)) - _dot(g, torch.ones_like(g))) <= 1e-6 * float(g.double().abs().sum())
    # every gradient entry sits at a maximum of its cluster
    nz = gx != 0
    assert torch.equal(x.detach()[nz], ref[cl][nz])
    # the arg-max indices of the whole grid, bit for bit against the oracle (smallest vertex wins a tie)
    from oracle import torch_ref as R
    from picassoplus_amd.mesh.pi_modules import mesh_pool3d
    torch.set_num_threads(16)
    y2, idx = mesh_pool3d.max_forward(x.detach(), vr, vm, vt_out)
    ref_y, ref_idx = R.maxpool_fwd(x.detach().cpu(), torch.from_numpy(vt_replace), torch.from_numpy(vt_map), nvo)
    assert np.array_equal(idx.cpu().numpy(), ref_idx.numpy()), "max_index differs from the oracle"
    assert np.array_equal(y2.cpu().numpy(), ref_y.numpy())
    del ref_y, ref_idx, y2, idx

    ya = pool3d.avgPool(x, vr, vm, vt_out)
    (gxa,) = torch.autograd.grad(ya, x, g)
    cnt = torch.zeros(nvo, device=cuda).index_add_(0, cl, torch.ones(nv, device=cuda))
    ref_a = torch.zeros(nvo, C, device=cuda, dtype=torch.float64).index_add_(0, cl, x.detach().double()) / cnt[:, None]
    assert float((ya.detach().double() - ref_a).abs().max()) <= 1e-5 * float(ref_a.abs().max())
    assert float((gxa - g[cl] / cnt[cl][:, None]).abs().max()) <= 1e-6 * float(g.abs().max())

    c = ya.detach().clone().requires_grad_(True)
    u = unpool3d.interpolate(c, vr, vm)
    gf = torch.randn(nv, C, device=cuda, generator=gen)
    (gc,) = torch.autograd.grad(u, c, gf)
    assert torch.equal(u.detach(), c.detach()[cl])                          # unpool copies
    back = pool3d.avgPool(u.detach(), vr, vm, vt_out)                      # avg_pool(unpool(y)) = y
    assert float((back - c.detach()).abs().max()) <= 2e-6 * float(c.detach().abs().max())
    ref_gc = torch.zeros(nvo, C, device=cuda, dtype=torch.float64).index_add_(0, cl, gf.double())
    assert float((gc.double() - ref_gc).abs().max()) <= 1e-5 * float(ref_gc.abs().max())
    torch.cuda.synchronize()


@pytest.mark.parametrize("ci,co", [(64, 64), (128, 128)])
def test_dense_tail_full_size_adjoints_and_sample_parity(cuda, ci, co):
    """The pointwise tail on 2.4 M rows: without activation y = x W + b is linear, so <y - b, g> = <x, gx> = <W, gW>
    and gb = column sums of g; with ReLU a random sample of rows is checked against the float64 oracle and the bit
    mask against the output."""
    from oracle import torch_ref
    from picassoplus_amd.mesh.pi_modules import dense
    say("case dense tail full size", ci, co)
    N = 2_400_000
    gen = torch.Generator(device=cuda).manual_seed(ci)
    x = torch.randn(N, ci, device=cuda, generator=gen)
    w = torch.randn(ci, co, device=cuda, generator=gen) / ci ** 0.5
    b = torch.randn(co, device=cuda, generator=gen)
    g = torch.randn(N, co, device=cuda, generator=gen)
    y = dense.dense_tail_forward(x, w, b, False)
    gx, gw, gb = dense.dense_tail_backward(g, x, w, None)
    lhs = _dot(y, g) - _dot(b[None, :].expand_as(g), g)
    scale = float(y.double().norm() * g.double().norm())
    _adjoint_ok(lhs, _dot(x, gx), scale, "dense <y-b,g> = <x,gx>")
    _adjoint_ok(lhs, _dot(w, gw), scale, "dense <y-b,g> = <W,gW>")
    assert_close(gb, g.double().sum(0).cpu().numpy(), "dense grad_bias")
    del y, gx
    yr, bits = dense.dense_tail_forward(x, w, b, True, with_bits=True)
    cols = torch.arange(co, device=cuda)
    pick = torch.randint(0, N, (4096,), device=cuda, generator=gen)
    assert torch.equal(((bits[pick][:, cols // 32] >> (cols % 32)) & 1).bool(), yr[pick] > 0)
    ref = torch_ref.dense_tail_fwd(x[pick].double().cpu(), w.double().cpu(), b.double().cpu(), True)
    assert_close(yr[pick], ref.numpy(), "dense forward sample")
    gxr, gwr, gbr = dense.dense_tail_backward(g, x, w, None, relu_bits=bits)
    rx, _, _ = torch_ref.dense_tail_bwd(g[pick].double().cpu(), x[pick].double().cpu(), w.double().cpu(),
                                        yr[pick].double().cpu())
    assert_close(gxr[pick], rx.numpy(), "dense grad_input sample")
    # the weight gradient of the masked pass, on the GPU in float64 from the same mask
    gz = torch.where(yr > 0, g, torch.zeros_like(g)).double()
    assert_close(gwr, (x.double().t() @ gz).cpu().numpy(), "dense grad_weight")
    assert_close(gbr, gz.sum(0).cpu().numpy(), "dense grad_bias (masked)")


def test_config_sphere_v2f_then_f2v_forward(cuda):
    """The single-mesh configuration: jittered icosphere of level 5 (10 242 vertices, 20 480 facets), one V2F
    convolution 32 -> 64 then one F2V convolution 64 -> 64, degree 3, Uniform(-1, 1) features, Xavier-uniform
    weights, forward only -- modules on the GPU against the float64 oracle composition."""
    from oracle import torch_ref as R
    from picassoplus_amd.mesh import layers
    say("case sphere level 5, V2F then F2V")
    mesh = S.sphere_workload(seed=1000, level=5)
    v, f = mesh["vertex"], mesh["face"]
    nv, nf = v.shape[0], f.shape[0]
    assert (nv, nf) == (10242, 20480)
    rng = np.random.default_rng(1000)
    x = rng.uniform(-1, 1, (nv, 32))
    normal, _ = S.triangle_normals_areas(v, f)
    nfc = S.vertex_facet_count(f, np.arange(nv), nv).astype(np.int32)
    torch.manual_seed(1000)
    v2f = layers.V2FConv3d(32, 64, 3, with_bn=False).to(cuda)
    f2v = layers.F2VConv3d(64, 64, 3, with_bn=False).to(cuda)
    with torch.no_grad():
        for m in (v2f, f2v):
            for p in m.parameters():
                if p.dim() > 1 and p.numel() > p.shape[-1]:
                    torch.nn.init.xavier_uniform_(p.view(p.shape[0], -1) if p.dim() == 3 else p)
            m.biases.uniform_(-0.1, 0.1)
        face, ident = dev(f, cuda), torch.arange(nv, dtype=torch.int32, device=cuda)
        coeff = sph_harm_values(dev(normal.astype(np.float32), cuda), 3)
        y = f2v(v2f(dev(x.astype(np.float32), cuda), face), face, dev(nfc, cuda), ident, coeff)
    torch.cuda.synchronize()
    T64 = lambda t: t.detach().cpu().double()
    f64, x64 = torch.from_numpy(f), torch.from_numpy(x.astype(np.float32)).double()
    spatial = (R.sph_harm(torch.eye(3, dtype=torch.float64), 3) @ T64(v2f.spatial_weights)).reshape(3, 32, 1)
    h = torch.relu(R.v2f_fwd(x64, spatial, f64) @ T64(v2f.depth_weights) + T64(v2f.biases))
    c64 = R.sph_harm(torch.from_numpy(normal.astype(np.float32)).double(), 3)
    h = R.f2v_fwd(h, T64(f2v.spatial_weights), c64, f64, torch.from_numpy(nfc), torch.arange(nv, dtype=torch.int32))
    ref = torch.relu(h @ T64(f2v.depth_weights) + T64(f2v.biases))
    assert float(ref.abs().max()) > 0
    assert_close(y, ref.numpy(), "sphere configuration output")


def test_config_shapes_block_forward_backward(cuda):
    """The shapes configuration at full size (16 meshes, about 329 k facets, C = 64, three texture points per
    facet): y = F2V(V2F(X) + F2F(texture(X))) with dL/dy ~ N(0, 1); output and the gradients of X and of the
    three filters against the float64 oracle."""
    from oracle import torch_ref as R
    from picassoplus_amd.mesh.pi_modules import texture
    say("case shapes block at full size")
    mesh = S.shapes_workload(seed=2000, n_meshes=16)
    v, f = mesh["vertex"], mesh["face"]
    nv, nf, C, L = v.shape[0], f.shape[0], 64, 3
    rng = np.random.default_rng(2000)
    normal, _ = S.triangle_normals_areas(v, f)
    counts, bary, _ = S.texture_points(rng, nf, np.full(nf, 3, np.int32))
    bary = bary.astype(np.float32)
    nfc = np.maximum(S.vertex_facet_count(f, np.arange(nv), nv), 1).astype(np.int32)
    x = rng.uniform(-1, 1, (nv, C)).astype(np.float32)
    w_v2f = S.xavier_uniform(rng, (3, C, 1), C, 3 * C).astype(np.float32)
    w_f2f = S.xavier_uniform(rng, (C, C, 16), C * 16, C * 16).astype(np.float32)
    w_f2v = S.xavier_uniform(rng, (16, C, 1), C, 16 * C).astype(np.float32)
    gy = rng.normal(0, 1, (nv, C)).astype(np.float32)
    leaves = [dev(a, cuda).requires_grad_(True) for a in (x, w_v2f, w_f2f, w_f2v)]
    xg, wv, wf, wo = leaves
    face, cum = dev(f, cuda), torch.cumsum(dev(counts, cuda), 0, dtype=torch.int32)
    ident = torch.arange(nv, dtype=torch.int32, device=cuda)
    tex, sh = texture.interpolate(xg, face, dev(bary, cuda), cum, L)
    y = conv3d.facet2vertex(conv3d.vertex2facet(xg, wv, face) + conv3d.facet2facet(tex, wf, sh, cum), wo,
                            sph_harm_values(dev(normal.astype(np.float32), cuda), L), face, dev(nfc, cuda), ident)
    grads = torch.autograd.grad(y, leaves, dev(gy, cuda))
    torch.cuda.synchronize()
    say("  oracle (float64, CPU)")
    torch.set_num_threads(8)
    D = lambda a: torch.from_numpy(a).double()
    ref_leaves = [D(a).requires_grad_(True) for a in (x, w_v2f, w_f2f, w_f2v)]
    x64, wv64, wf64, wo64 = ref_leaves
    f64, cum64, b64 = torch.from_numpy(f), torch.from_numpy(np.cumsum(counts).astype(np.int32)), D(bary)
    tex64 = R.texture_fwd(x64, f64, b64, cum64)
    y64 = R.f2v_fwd(R.v2f_fwd(x64, wv64, f64) + R.f2f_fwd(tex64, wf64, R.sph_harm(b64, L), cum64), wo64,
                    R.sph_harm(D(normal.astype(np.float32)), L), f64, torch.from_numpy(nfc), torch.arange(nv, dtype=torch.int32))
    ref_grads = torch.autograd.grad(y64, ref_leaves, D(gy))
    assert_close(y, y64.detach().numpy(), "shapes block output")
    for name, g, r in zip(("X", "V2F filter", "F2F filter", "F2V filter"), grads, ref_grads):
        assert_close(g, r.numpy(), "shapes block gradient of " + name)


def test_point_conv_full_size_adjoints_and_sample_parity(cuda):
    """The bench's point-cloud workload (every 16th vertex of the scene batch, spherical-harmonic graph of at most 16
    neighbours, 128 channels): the fuzzy point convolution is linear in its input and in its filter, so
    <g, conv(x, w)> = <x, grad_x> = <w, grad_w>; a sample of output rows against the float64 oracle; the graph's
    invariants (counts within the limit, every point its own neighbour, pairs sorted by query)."""
    from oracle import point_ref
    from picassoplus_amd.point import utils as PU
    from picassoplus_amd.point.pi_modules import conv3d as pconv
    say("case point conv full size")
    mesh = S.scene_workload(seed=3000, n_rooms=8, scale=1.0)
    nv_in = np.asarray(mesh["nv_in"], np.int64)
    start = np.concatenate([[0], np.cumsum(nv_in)])
    keep = np.concatenate([np.arange(start[b], start[b + 1], 16) for b in range(len(nv_in))])
    nv = np.array([len(np.arange(start[b], start[b + 1], 16)) for b in range(len(nv_in))], np.int32)
    xyz = dev(np.ascontiguousarray(mesh["vertex"][keep], dtype=np.float32), cuda)
    NV = dev(nv, cuda)
    C, L, limit, radius = 128, 3, 16, 0.18
    nn_cnt, nn_idx, nn_dst, filt_idx, filt_coeff = PU.build_sphere_harmonics(xyz, xyz, NV, NV, radius, L=L, nn_uplimit=limit)
    Np, P, T = xyz.shape[0], nn_idx.shape[0], filt_idx.shape[1]
    cnt = nn_cnt.cpu().numpy()
    idx = nn_idx.cpu().numpy()
    assert cnt.sum() == P and cnt.min() >= 1 and cnt.max() <= limit and T == (L + 1) ** 2 + 1
    assert np.all(np.diff(idx[:, 0]) >= 0) and np.array_equal(np.bincount(idx[:, 0], minlength=Np), cnt)
    first = np.concatenate([[0], np.cumsum(cnt)[:-1]])
    sample_of = np.repeat(np.arange(len(nv)), nv)
    assert np.array_equal(sample_of[idx[:, 0]], sample_of[idx[:, 1]])           # neighbours stay inside the sample
    assert bool((nn_dst < radius).all())
    gen = torch.Generator(device=cuda).manual_seed(11)
    x = torch.randn(Np, C, device=cuda, generator=gen).requires_grad_(True)
    w = (torch.randn(T, C, 1, device=cuda, generator=gen) / 4).requires_grad_(True)
    g = torch.randn(Np, C, device=cuda, generator=gen)
    y = pconv.fuzzyconv3d(x, w, nn_cnt, nn_idx, filt_idx, filt_coeff)
    gx, gw = torch.autograd.grad(y, [x, w], g)
    lhs = _dot(g, y.detach())
    scale = float(g.double().norm() * y.detach().double().norm())
    _adjoint_ok(lhs, _dot(x.detach(), gx), scale, "point conv: <g, y> = <x, gx>")
    _adjoint_ok(lhs, _dot(w.detach(), gw), scale, "point conv: <g, y> = <w, gw>")
    # sampled rows against the oracle (each row needs only its own pairs)
    rng = np.random.default_rng(12)
    rows = np.sort(rng.choice(Np, 400, replace=False))
    fi, fc = filt_idx.cpu().numpy(), filt_coeff.cpu().numpy().astype(np.float64)
    xs, ws = x.detach().cpu().numpy().astype(np.float64), w.detach().cpu().numpy().astype(np.float64)
    sel = np.concatenate([np.arange(first[r], first[r] + cnt[r]) for r in rows])
    sub_idx = idx[sel].copy()
    sub_idx[:, 0] = np.repeat(np.arange(len(rows)), cnt[rows])
    ref = point_ref.conv_fwd(xs, ws, cnt[rows], sub_idx, fi[sel], fc[sel])
    assert_close(y.detach()[torch.from_numpy(rows).to(cuda)], ref, "point conv sampled rows")


def test_decimation_full_size_invariants(cuda):
    """The scene batch decimated to a quarter of its vertices: the maps' invariants (A.5 of the pooling ops' contract),
    facets that reference live output vertices only, no degenerate facet left, the sample counts, a second run
    bit-equal to the first, and max pooling over the maps equal to a brute-force maximum over the clusters on a sample."""
    from picassoplus_amd.mesh.pi_modules import decimate as D
    say("case decimation full size")
    mesh = S.scene_workload(seed=3000, n_rooms=8, scale=1.0)
    vertex, face = dev(mesh["vertex"].astype(np.float32), cuda), dev(mesh["face"].astype(np.int32), cuda)
    nv_in, mf_in = dev(mesh["nv_in"].astype(np.int32), cuda), dev(mesh["mf_in"].astype(np.int32), cuda)
    nv_out = (nv_in // 4).to(torch.int32)
    geometry = D.compute_triangle_geometry_(vertex, face)
    out = D.mesh_decimation_(vertex, face, geometry, nv_in, mf_in, nv_out)
    again = D.mesh_decimation_(vertex, face, geometry, nv_in, mf_in, nv_out)
    for a, b in zip(out, again):
        assert torch.equal(a, b)
    v2, f2, g2, nv2, mf2, rep, vmap = out
    Nv, Nv2 = vertex.shape[0], v2.shape[0]
    assert int(nv2.sum()) == Nv2 and int(mf2.sum()) == f2.shape[0] and tuple(g2.shape) == (f2.shape[0], 5)
    # every sample reaches its target (a few vertices below it: vertices that lose their last facet are dropped too)
    assert bool((nv2 <= nv_in).all())
    assert bool((nv2.double() <= nv_out.double()).all()) and bool((nv2.double() >= 0.99 * nv_out.double() - 8).all())
    assert int(f2.min()) >= 0 and int(f2.max()) < Nv2
    fl = f2.long()
    assert not bool(((fl[:, 0] == fl[:, 1]) | (fl[:, 0] == fl[:, 2]) | (fl[:, 1] == fl[:, 2])).any())
    r, m = rep.cpu().numpy().astype(np.int64), vmap.cpu().numpy().astype(np.int64)
    contracted = r < 0
    target = np.where(contracted, -r, np.arange(Nv))
    assert np.all(r[target] >= 0)                                  # a representative is not contracted itself
    assert np.array_equal(np.bincount(target, minlength=Nv)[~contracted] - 1, r[~contracted])   # member counts
    assert np.all(m[contracted] == -1)
    live = m >= 0
    assert np.array_equal(np.sort(m[live]), np.arange(Nv2)) and np.all(np.diff(m[live]) > 0)   # ascending numbering
    # pooling over the maps on a sample of coarse vertices
    x = torch.randn(Nv, 8, device=cuda, generator=torch.Generator(device=cuda).manual_seed(3))
    pooled = pool3d.maxPool(x, rep, vmap, v2)
    coarse = m[target]                                             # coarse row of every input vertex (-1: dropped cluster)
    rng = np.random.default_rng(4)
    pick = rng.choice(Nv2, 300, replace=False)
    xs = x.cpu().numpy()
    order = np.argsort(coarse, kind="stable")
    lo = np.searchsorted(coarse[order], pick, side="left")
    hi = np.searchsorted(coarse[order], pick, side="right")
    want = np.stack([xs[order[a:b]].max(0) for a, b in zip(lo, hi)])
    assert np.array_equal(pooled[torch.from_numpy(pick).to(cuda)].cpu().numpy(), want)


@pytest.mark.parametrize("level,C", [(0, 32), (3, 256)])
def test_hierarchy_level_full_size(cuda, level, C):
    """The finest (2.1 M facets, width 32) and the coarsest (32 768 facets, width 256) level of the hierarchy
    workload at the bench's sizes: the three convolutions through adjoint identities, oracle parity on sampled
    facets / vertices, and the facet2facet filter gradient element by element.  These are the kernel instances the
    scene batch does not reach (half-empty 64-column tiles at width 32, four blocks of 64 output channels at 256)."""
    from oracle import torch_ref as R
    torch.set_num_threads(16)
    cells = 1024 >> level
    say("case hierarchy level", level, "width", C, "cells", cells)
    rng = np.random.default_rng(5000 + level)
    h = float(1 << level)
    v, f = S.grid_patch(rng, cells, cells, (0, 0, 0), (h, 0, 0), (0, h, 0), flip_frac=0.5)
    v = v + rng.normal(0, 0.1 * h, v.shape) * np.array([1.0, 1.0, 0.2])
    nv, nf = v.shape[0], f.shape[0]
    assert nf == 2 * cells * cells
    normal, _ = S.triangle_normals_areas(v, f)
    counts, bary, _ = S.texture_points(rng, nf, rng.integers(1, 4, nf).astype(np.int32))
    T = int(counts.sum())
    face, cum = dev(f, cuda), torch.cumsum(dev(counts, cuda), 0, dtype=torch.int32)
    sh = sph_harm_values(dev(bary.astype(np.float32), cuda), 3)
    coeff = sph_harm_values(dev(normal.astype(np.float32), cuda), 3)
    nfc_np = np.maximum(S.vertex_facet_count(f, np.arange(nv), nv), 1).astype(np.int32)
    nfc, ident = dev(nfc_np, cuda), torch.arange(nv, dtype=torch.int32, device=cuda)
    gen = torch.Generator(device=cuda).manual_seed(50 + level)

    # facet2facet C -> C
    tex = torch.rand(T, C, device=cuda, generator=gen).mul_(2).sub_(1).requires_grad_(True)
    w = dev(S.xavier_uniform(rng, (C, C, 16), C * 16, C * 16).astype(np.float32), cuda).requires_grad_(True)
    g = torch.randn(nf, C, device=cuda, generator=gen)
    out = conv3d.facet2facet(tex, w, sh, cum)
    gtex, gw = torch.autograd.grad(out, [tex, w], g)
    torch.cuda.synchronize()
    lhs, scale = _dot(out, g), float(out.double().norm() * g.double().norm())
    _adjoint_ok(lhs, _dot(tex, gtex), scale, "<f2f(tex), g> = <tex, grad_texture>")
    _adjoint_ok(lhs, _dot(w, gw), scale, "<f2f(tex), g> = <W, grad_filter>")
    pick = np.sort(rng.choice(nf, 600, replace=False))
    start = np.concatenate([[0], np.cumsum(counts)])[:-1]
    rows = np.concatenate([np.arange(start[i], start[i] + counts[i]) for i in pick]).astype(np.int64)
    rows_t, pick_t = torch.from_numpy(rows).to(cuda), torch.from_numpy(pick).to(cuda)
    w64 = w.detach().cpu().numpy().astype(np.float64)
    sub_tex, sub_sh = tex.detach()[rows_t].cpu().numpy().astype(np.float64), sh[rows_t].cpu().numpy().astype(np.float64)
    sub_cum = np.cumsum(counts[pick]).astype(np.int32)
    ref_out = loops.f2f_fwd(sub_tex, w64, sub_sh, sub_cum)
    ref_gtex, _ = loops.f2f_bwd(g[pick_t].cpu().numpy().astype(np.float64), sub_tex, w64, sub_sh, sub_cum)
    tag = " (hierarchy level %d)" % level
    assert_close(out.detach()[pick_t], ref_out, "f2f out, sampled facets" + tag)
    assert_close(gtex[rows_t], ref_gtex, "f2f grad_texture, sampled facets" + tag)
    ref_gw = R.f2f_bwd_filter_pointwise(g.cpu().double(), tex.detach().cpu().double(), sh.cpu().double(), cum.cpu())
    assert_close(gw, ref_gw.numpy(), "f2f grad_filter, element by element" + tag)
    del out, gtex, gw, ref_gw, tex

    # facet2vertex C -> C and vertex2facet C -> C
    x = torch.randn(nf, C, device=cuda, generator=gen).requires_grad_(True)
    wv = dev(S.xavier_uniform(rng, (16, C, 1), C, 16 * C).astype(np.float32), cuda).requires_grad_(True)
    gv = torch.randn(nv, C, device=cuda, generator=gen)
    y = conv3d.facet2vertex(x, wv, coeff, face, nfc, ident)
    gx, gwv = torch.autograd.grad(y, [x, wv], gv)
    torch.cuda.synchronize()
    lhs, scale = _dot(y, gv), float(y.double().norm() * gv.double().norm())
    _adjoint_ok(lhs, _dot(x, gx), scale, "<f2v(x), g> = <x, grad_input>")
    _adjoint_ok(lhs, _dot(wv, gwv), scale, "<f2v(x), g> = <filter, grad_filter>")
    f_np = f.astype(np.int64)
    x_np, wv_np, cf_np = (a.detach().cpu().numpy().astype(np.float64) for a in (x, wv, coeff))
    pick_v = np.sort(rng.choice(nv, 1000, replace=False))
    is_pick = np.zeros(nv, bool)
    is_pick[pick_v] = True
    around = np.nonzero(is_pick[f_np].any(1))[0]
    sub = loops.f2v_fwd(x_np[around], wv_np, cf_np[around], f[around].astype(np.int32), nfc_np, np.arange(nv, dtype=np.int32))
    assert_close(y.detach()[torch.from_numpy(pick_v).to(cuda)], sub[pick_v], "f2v out, sampled vertices" + tag)
    pick_f = np.sort(rng.choice(nf, 1000, replace=False))
    sub_gin, _ = loops.f2v_bwd(gv.cpu().numpy().astype(np.float64), x_np[pick_f], wv_np, cf_np[pick_f],
                               f[pick_f].astype(np.int32), nfc_np, np.arange(nv, dtype=np.int32))
    assert_close(gx[torch.from_numpy(pick_f).to(cuda)], sub_gin, "f2v grad_input, sampled facets" + tag)
    _, ref_gwv = R.f2v_bwd(gv.cpu().double(), x.detach().cpu().double(), wv.detach().cpu().double(), coeff.cpu().double(),
                           face.cpu(), nfc.cpu(), ident.cpu())
    assert_close(gwv, ref_gwv.numpy(), "f2v grad_filter, element by element" + tag)
    del y, gx, x

    xv = torch.randn(nv, C, device=cuda, generator=gen).requires_grad_(True)
    w3 = torch.randn(3, C, 1, device=cuda, generator=gen).requires_grad_(True)
    gf = torch.randn(nf, C, device=cuda, generator=gen)
    z = conv3d.vertex2facet(xv, w3, face)
    gxv, gw3 = torch.autograd.grad(z, [xv, w3], gf)
    torch.cuda.synchronize()
    lhs, scale = _dot(z, gf), float(z.double().norm() * gf.double().norm())
    _adjoint_ok(lhs, _dot(xv, gxv), scale, "<v2f(x), g> = <x, grad_input>")
    _adjoint_ok(lhs, _dot(w3, gw3), scale, "<v2f(x), g> = <filter, grad_filter>")
    sub_z = loops.v2f_fwd(xv.detach().cpu().numpy().astype(np.float64), w3.detach().cpu().numpy().astype(np.float64), f[pick_f])
    assert_close(z.detach()[torch.from_numpy(pick_f).to(cuda)], sub_z, "v2f out, sampled facets" + tag)
