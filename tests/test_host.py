"""Host-side checks that need no GPU: the C ABI library loads and exports what the header
declares, argument errors surface as RuntimeError the way the reference's CHECK_INPUT does,
the modules keep the reference's signatures / parameter names, the generators obey the index
invariants the kernels rely on."""
import inspect
import os
import re
import subprocess
import sys

import numpy as np
import pytest
import torch

from picassoplus_amd import _lib, synthetic as S
from picassoplus_amd.mesh import layers
from picassoplus_amd.mesh.pi_modules import conv3d, mesh_conv3d, mesh_pool3d, mesh_unpool3d, pool3d, texture, unpool3d

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "picasso_mesh.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pmesh_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = header_symbols()
    assert len(names) >= 24
    for n in names:
        assert hasattr(lib, n), "libpicasso_mesh.so lacks %s" % n
    assert sorted(_lib.SIGNATURES) == names          # the ctypes table covers the header, no more, no less
    assert lib.pmesh_abi_version() == _lib.ABI_VERSION
    assert lib.pmesh_last_error() == b""


def test_size_queries_are_host_only():
    assert _lib.query("pmesh_v2f_bwd_workspace_bytes", 64, 1) == 1024 * 3 * 64 * 4
    assert _lib.query("pmesh_f2v_bwd_workspace_bytes", 64, 1, 16) == 1024 * 16 * 64 * 4
    assert _lib.query("pmesh_f2f_bwd_workspace_bytes", 64, 64, 16) == 256 * 64 * 64 * 16 * 4 + 256    # partials + flag
    assert _lib.query("pmesh_f2f_fwd_workspace_bytes", 64, 64, 16) == 64 * 2 * 3 * 64 * 16
    assert _lib.query("pmesh_f2f_fwd_workspace_bytes", 3, 64, 16) == 4 * 2 * 3 * 64 * 16      # channels padded to 4
    assert _lib.query("pmesh_f2f_fwd_workspace_bytes", 3, 64, 9) == 0
    assert _lib.query("pmesh_facet_order_workspace_bytes", 1000) >= 3 * 1000 * 4
    assert _lib.query("pmesh_vertex_csr_workspace_bytes", 1000, 500) >= 3 * 3000 * 4
    assert _lib.query("pmesh_cluster_csr_workspace_bytes", 1000, 250) >= 3 * 1000 * 4


def test_argument_errors_without_launching():
    lib = _lib.load()
    # bad dimensions are rejected before any device work, with a message
    assert lib.pmesh_v2f_fwd(None, None, None, None, 10, 10, 0, 1, None) != 0
    assert b"bad channel counts" in lib.pmesh_last_error()
    assert lib.pmesh_f2f_fwd(None, None, None, None, None, None, None, 0, 10, 10, 4, 4, 51, None) != 0
    assert b"maximum of 50" in lib.pmesh_last_error()
    assert lib.pmesh_sph_harm(None, None, 5, 6, None) != 0
    assert lib.pmesh_pool_max_bwd(None, None, None, None, None, -1, 2, 4, None) != 0
    assert lib.pmesh_texture_fwd(None, None, None, None, None, None, 4, 2, 6, 8, 3, None) != 0
    assert b"null pointer" in lib.pmesh_last_error()
    assert lib.pmesh_texture_bwd(None, None, None, None, None, None, 4, 2, -1, 8, None) != 0
    assert lib.pmesh_texture_fwd(None, None, None, None, None, None, 4, 2, 0, 8, 3, None) == 0
    assert lib.pmesh_facet_frame(None, None, None, None, None, 4, 2, 2, 3, None) != 0
    assert lib.pmesh_facet_frame(None, None, None, None, None, 4, 2, 3, 3, None) == 0      # nothing asked for
    # empty problems succeed without touching the (null) pointers
    assert lib.pmesh_v2f_fwd(None, None, None, None, 0, 0, 8, 1, None) == 0
    assert lib.pmesh_last_error() == b""


def test_cpu_tensors_are_refused_like_the_reference():
    x, filt, face = torch.zeros(4, 8), torch.zeros(3, 8, 1), torch.zeros(2, 3, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        conv3d.vertex2facet(x, filt, face)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        conv3d.facet2vertex(x, filt, torch.zeros(4, 3), face, torch.zeros(4, dtype=torch.int32), torch.zeros(4, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        conv3d.facet2facet(x, torch.zeros(8, 8, 16), torch.zeros(4, 16), torch.zeros(2, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        pool3d.maxPool(x, torch.zeros(4, dtype=torch.int32), torch.zeros(4, dtype=torch.int32), torch.zeros(2, 3))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        pool3d.avgPool(x, torch.zeros(4, dtype=torch.int32), torch.zeros(4, dtype=torch.int32), torch.zeros(2, 3))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        unpool3d.interpolate(x, torch.zeros(4, dtype=torch.int32), torch.zeros(4, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        layers.SphHarmCoeff(3)(torch.eye(3))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        texture.interpolate(x, face, torch.zeros(4, 3), torch.zeros(2, dtype=torch.int32))


def test_native_module_surface_matches_reference_extensions():
    # the three pybind modules of the reference and their function names / arities
    assert [len(inspect.signature(getattr(mesh_conv3d, n)).parameters) for n in
            ("vertex2facet_forward", "vertex2facet_backward", "facet2vertex_forward", "facet2vertex_backward",
             "facet2facet_forward", "facet2facet_backward")] == [3, 4, 6, 7, 4, 5]
    assert [len(inspect.signature(getattr(mesh_pool3d, n)).parameters) for n in
            ("max_forward", "avg_forward", "avg_backward")] == [4, 4, 4]
    assert list(inspect.signature(mesh_pool3d.max_backward).parameters)[:3] == ["grad_output", "input", "max_index"]
    assert [len(inspect.signature(getattr(mesh_unpool3d, n)).parameters) for n in ("forward", "backward")] == [3, 4]
    assert list(inspect.signature(conv3d.facet2facet).parameters) == ["textureIn", "filter", "baryCoeff", "numTexture"]
    assert list(inspect.signature(conv3d.vertex2facet).parameters) == ["input", "filter", "face"]
    assert list(inspect.signature(conv3d.facet2vertex).parameters) == ["input", "filter", "coeff", "face", "nfCount", "vtMap"]
    assert list(inspect.signature(pool3d.maxPool).parameters) == ["input", "vt_replace", "vt_map", "vt_out"]
    assert list(inspect.signature(pool3d.avgPool).parameters) == ["input", "vt_replace", "vt_map", "vt_out"]
    assert list(inspect.signature(unpool3d.interpolate).parameters) == ["input", "vt_replace", "vt_map"]


def test_module_signatures_and_state_dict_keys():
    sig = lambda cls: list(inspect.signature(cls.__init__).parameters)[1:]
    assert sig(layers.F2FConv3d) == ["in_channels", "out_channels", "spharm_L", "use_xavier", "stddev",
                                     "activation_fn", "with_bn", "bn_momentum"]
    sep = ["in_channels", "out_channels", "spharm_L", "depth_multiplier", "use_xavier", "stddev",
           "activation_fn", "with_bn", "bn_momentum"]
    assert sig(layers.V2FConv3d) == sep and sig(layers.F2VConv3d) == sep
    assert sig(layers.V2VConv3d) == ["in_channels", "dual_out_channels", "spharm_L", "dual_depth_multiplier",
                                     "use_xavier", "stddev", "activation_fn", "with_bn", "bn_momentum"]
    assert list(inspect.signature(layers.F2FConv3d.forward).parameters)[1:] == ["input_texture", "bary_coeff", "num_texture"]
    assert list(inspect.signature(layers.V2FConv3d.forward).parameters)[1:] == ["inputs", "face"]
    assert list(inspect.signature(layers.F2VConv3d.forward).parameters)[1:] == ["inputs", "face", "nf_count", "vt_map", "filt_coeff"]
    assert list(inspect.signature(layers.Pool3d.forward).parameters)[1:] == ["inputs", "vt_replace", "vt_map", "vt_out"]
    assert list(inspect.signature(layers.Unpool3d.forward).parameters) == ["inputs", "vt_replace", "vt_map"]

    bn = ["BatchNorm.weight", "BatchNorm.bias", "BatchNorm.running_mean", "BatchNorm.running_var", "BatchNorm.num_batches_tracked"]
    m = layers.F2FConv3d(3, 32, 3)
    assert sorted(m.state_dict()) == sorted(["weights", "biases"] + bn)
    assert tuple(m.weights.shape) == (32, 3, 16) and tuple(m.biases.shape) == (1, 32) and m.BatchNorm.eps == 0.001
    m = layers.V2FConv3d(8, 12, 3, depth_multiplier=2)
    assert sorted(m.state_dict()) == sorted(["spatial_weights", "depth_weights", "biases"] + bn)
    assert tuple(m.spatial_weights.shape) == (16, 16) and tuple(m.depth_weights.shape) == (16, 12)
    m = layers.F2VConv3d(8, 12, 2, depth_multiplier=2)
    assert tuple(m.spatial_weights.shape) == (9, 8, 2) and tuple(m.depth_weights.shape) == (16, 12)
    m = layers.V2VConv3d(8, [16, 24], 3, [1, 2], with_bn=False)
    assert sorted(m.state_dict()) == sorted(p + k for p in ("V2F_conv3d.", "F2V_conv3d.")
                                            for k in ("spatial_weights", "depth_weights", "biases"))
    m = layers.PerItemConv3d(8, 4)
    assert sorted(m.state_dict()) == sorted(["weights", "biases"] + bn) and tuple(m.weights.shape) == (8, 4)
    assert sorted(layers.BuildF2VCoeff(5).state_dict()) == ["centers"]
    with pytest.raises(ValueError):
        layers.Pool3d("median")(None, None, None, None)
    # truncated-normal initialiser when xavier is off
    torch.manual_seed(0)
    w = layers.F2VConv3d(64, 64, 3, use_xavier=False, stddev=1e-3).spatial_weights
    assert float(w.detach().abs().max()) <= 2.0 and float(w.detach().std()) < 2e-3


def test_global_pool_cpu():
    x = torch.tensor([[1., 5.], [3., 2.], [0., 7.], [4., 4.], [9., -1.]])
    nv = torch.tensor([2, 3])
    assert torch.allclose(layers.GlobalPool3d("avg")(x, nv), torch.tensor([[2., 3.5], [13 / 3, 10 / 3]]))
    val, arg = layers.GlobalPool3d("max")(x, nv)
    assert val.tolist() == [[3., 5.], [9., 7.]] and arg.tolist() == [[1, 0], [4, 2]]


# ------------------------------------------------------------------ generators
def test_mesh_generators():
    v, f = S.icosphere(5)
    assert v.shape == (10242, 3) and f.shape == (20480, 3) and f.dtype == np.int32
    assert np.allclose(np.linalg.norm(v, axis=1), 1) and np.bincount(f.reshape(-1)).min() >= 5
    v, f = S.torus(12, 8)
    assert v.shape[0] == 96 and f.shape[0] == 192 and set(np.bincount(f.reshape(-1))) == {6}
    w = S.shapes_workload(seed=2000, n_meshes=3)
    assert w["face"].max() == w["vertex"].shape[0] - 1 and w["mf_in"].sum() == w["face"].shape[0]
    offs = np.concatenate([[0], np.cumsum(w["nv_in"])])
    fo = np.concatenate([[0], np.cumsum(w["mf_in"])])
    for i in range(3):                                  # facets of sample i only use vertices of sample i
        blk = w["face"][fo[i]:fo[i + 1]]
        assert blk.min() >= offs[i] and blk.max() < offs[i + 1]
    v, f = S.room(np.random.default_rng(0), scale=0.02)
    assert f.min() == 0 and f.max() == v.shape[0] - 1
    assert (f[:, 0] != f[:, 1]).all() and (f[:, 1] != f[:, 2]).all() and (f[:, 0] != f[:, 2]).all()
    w = S.plane_workload(n=33)
    assert w["vertex"].shape[0] == 33 * 33 and w["face"].shape[0] == 2 * 32 * 32


@pytest.mark.parametrize("spatial", [True, False])
def test_cluster_map_invariants(spatial):
    rng = np.random.default_rng(5)
    nv = 20000
    r, m, nvo = S.cluster_maps(rng, nv, spatial=spatial, orphan_frac=0.03)
    members = r < 0
    reps = -r[members]
    assert (r[reps] > 0).all()                          # flat: a representative is never a member
    assert 0 not in set(reps.tolist())                  # vertex 0 never represents others
    assert (m[members] == -1).all()
    assert np.array_equal(np.bincount(reps, minlength=nv)[r > 0], r[r > 0])   # value = number of other members
    kept = m >= 0
    assert nvo == kept.sum() and np.array_equal(m[kept], np.arange(nvo))      # ascending, dense
    sizes = r[r >= 0] + 1
    assert sizes.min() >= 1 and sizes.max() <= 12 and 3.5 < sizes.mean() < 4.5 and sizes.sum() == nv


def test_hierarchy_workload_levels_and_maps():
    levels = S.hierarchy_workload(seed=1, cells=16, levels=3)
    assert [lv["vertex"].shape[0] for lv in levels] == [17 * 17, 9 * 9, 5 * 5, 3 * 3]
    assert [lv["face"].shape[0] for lv in levels] == [2 * 16 * 16, 2 * 8 * 8, 2 * 4 * 4, 2 * 2 * 2]
    for fine, coarse in zip(levels[:-1], levels[1:]):
        r, m, nvo = fine["vt_replace"], fine["vt_map"], fine["nv_out"]
        nv = fine["vertex"].shape[0]
        assert nvo == coarse["vertex"].shape[0] and fine["face"].max() == nv - 1
        members = r < 0
        reps = -r[members]
        assert (r[reps] > 0).all() and 0 not in set(reps.tolist()) and (m[members] == -1).all()
        assert np.array_equal(np.bincount(reps, minlength=nv)[r > 0], r[r > 0])
        kept = m >= 0
        assert np.array_equal(m[kept], np.arange(nvo))                         # ascending, dense
        assert (r[r >= 0] + 1).sum() == nv and (r[r >= 0] + 1).max() == 4
        # a coarse vertex sits among its members: within one fine cell (plus jitter) of their mean position
        rep_of = np.where(r < 0, -r, np.arange(nv))
        mean = np.zeros((nvo, 3))
        np.add.at(mean, m[rep_of], fine["vertex"])
        mean /= np.bincount(m[rep_of], minlength=nvo)[:, None]
        step = fine["vertex"][:, 0].max() / (np.sqrt(nv) - 1)
        assert np.abs(mean - coarse["vertex"])[:, :2].max() < 2.0 * step


def test_texture_points():
    rng = np.random.default_rng(6)
    counts, bary, owner = S.texture_points(rng, 100, rng.integers(0, 10, 100))
    assert bary.shape == (counts.sum(), 3) and np.allclose(bary.sum(1), 1) and (bary >= 0).all()
    assert np.array_equal(np.bincount(owner, minlength=100), counts)
    k = S.area_scaled_texture_counts(rng.random(1000))
    assert k.min() >= 1 and k.max() == 9


def test_bench_refuses_more_than_one_gpu():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode != 0 and "one GPU" in res.stderr


def test_adjacency_cache_discipline():
    """The cache of per-index-tensor arrays: an entry dies with its index tensor (weak references), inference
    tensors are accepted as keys, the least recently used entries go when the byte bound is passed, and an in-place
    change of an index tensor makes a new key.  Host-side logic only: the cached values here are CPU tensors."""
    import gc
    from picassoplus_amd.mesh import topology as T
    T.clear_cache()
    a = torch.arange(12, dtype=torch.int32)
    calls = []
    T.checked_once("x", (a,), (3,), lambda: calls.append(1))
    T.checked_once("x", (a,), (3,), lambda: calls.append(1))
    assert calls == [1] and T.cache_entries() == 1
    a.add_(1)                                         # version counter moved: a new key
    T.checked_once("x", (a,), (3,), lambda: calls.append(1))
    assert calls == [1, 1]
    del a
    gc.collect()
    assert T.cache_entries() == 0                     # entries went with their tensor
    with torch.inference_mode():
        b = torch.arange(6, dtype=torch.int32)
    assert b.is_inference()
    T.checked_once("x", (b,), (), lambda: calls.append(1))    # no version counter to read on this one
    assert T.cache_entries() == 1
    # byte bound: three arrays of 400 bytes against a bound of 1000
    old = T.MAX_BYTES
    try:
        T.MAX_BYTES = 1000
        T.clear_cache()
        owners = [torch.zeros(4, dtype=torch.int32) for _ in range(3)]
        for i, o in enumerate(owners):
            arr = torch.zeros(100, dtype=torch.int32)
            T._store(T._key("y", o), arr, (o,), (arr,))
        assert T.cache_entries() == 2 and T.cache_bytes() == 800
        assert T._lookup(T._key("y", owners[0])) is None and T._lookup(T._key("y", owners[2])) is not None
    finally:
        T.MAX_BYTES = old
        T.clear_cache()
    assert T.cache_bytes() == 0


@pytest.mark.parametrize("seed", range(8))
def test_host_vertex_clustering_matches_the_oracle(seed):
    """pmesh_cluster_vertices_host runs on host arrays (no device needed): the two greedy passes over the candidate
    edges, bit-exact against the oracle's statement of them."""
    import ctypes

    from oracle import decimate_ref
    rng = np.random.default_rng(seed)
    num, start = (300, 0) if seed % 2 else (120, 50)
    pairs = sorted({tuple(sorted(p)) for p in rng.integers(start, start + num, (4 * num, 2)).tolist() if p[0] != p[1]})
    order = rng.permutation(len(pairs))
    vi = np.ascontiguousarray(np.array(pairs, np.int32)[order, 0])
    vj = np.ascontiguousarray(np.array(pairs, np.int32)[order, 1])
    for budget in (0, 1, num // 5, num):
        got = np.zeros(start + num, np.int32)
        _lib.call("pmesh_cluster_vertices_host", vi.ctypes.data, vj.ctypes.data, len(vi), start, num, budget, got.ctypes.data)
        want = np.zeros(start + num, np.int32)
        decimate_ref.cluster_vertices(vi, vj, start, num, budget, want)
        assert np.array_equal(got, want)
        assert (got < 0).sum() <= budget
    with pytest.raises(RuntimeError):                       # an edge that leaves the sample's vertex range
        _lib.call("pmesh_cluster_vertices_host", vi.ctypes.data, vj.ctypes.data, len(vi), start, num // 2, num, got.ctypes.data)


def test_call_many_runs_independent_samples_on_threads_and_reports_a_failure():
    """_lib.call_many: the samples of a batch (disjoint vertex ranges of one vt_replace array) on a thread pool give what
    one call after the other gives; a failing call raises with the library's message of ITS thread."""
    import ctypes

    rng = np.random.default_rng(7)
    P = ctypes.c_void_p
    num, samples = 200, 6
    vi_all, vj_all, jobs = [], [], []
    for b in range(samples):
        pairs = sorted({tuple(sorted(p)) for p in rng.integers(b * num, (b + 1) * num, (3 * num, 2)).tolist() if p[0] != p[1]})
        perm = rng.permutation(len(pairs))
        vi_all.append(np.ascontiguousarray(np.array(pairs, np.int32)[perm, 0]))
        vj_all.append(np.ascontiguousarray(np.array(pairs, np.int32)[perm, 1]))
    one, many = np.zeros(samples * num, np.int32), np.zeros(samples * num, np.int32)
    for b in range(samples):
        _lib.call("pmesh_cluster_vertices_host", vi_all[b].ctypes.data, vj_all[b].ctypes.data, len(vi_all[b]), b * num, num, num // 3,
                  one.ctypes.data)
        jobs.append((P(vi_all[b].ctypes.data), P(vj_all[b].ctypes.data), len(vi_all[b]), b * num, num, num // 3, P(many.ctypes.data)))
    _lib.call_many("pmesh_cluster_vertices_host", jobs)
    assert np.array_equal(one, many) and (many < 0).sum() > 0
    seen = []
    _lib.set_call_hook(lambda name, phase: seen.append((name, phase)))
    try:
        _lib.call_many("pmesh_cluster_vertices_host", jobs[:2])
    finally:
        _lib.set_call_hook(None)
    assert seen == [("pmesh_cluster_vertices_host", "begin"), ("pmesh_cluster_vertices_host", "end")]
    bad = list(jobs)
    bad[3] = bad[3][:4] + (num // 2,) + bad[3][5:]          # the sample's range cut in half: its edges leave it
    with pytest.raises(RuntimeError, match="outside the sample's vertex range"):
        _lib.call_many("pmesh_cluster_vertices_host", bad)


def test_bf16_store_criterion_tells_rounding_from_truncation():
    """The slack the bf16 parity criterion grants the final store (2^-8 of each value) covers round-to-nearest and
    nothing more: the same exact results stored by truncation fail it."""
    import torch
    from util import assert_close_bf16_store
    rng = np.random.default_rng(5)
    ref = rng.uniform(0.5, 4.0, 20000) * rng.choice([-1.0, 1.0], 20000)
    as_f32 = torch.from_numpy(ref.astype(np.float32))
    rounded = as_f32.to(torch.bfloat16)
    truncated = (as_f32.view(torch.int32) & -65536).view(torch.float32)
    # the criterion's own tolerance set to (almost) nothing: only the store's rounding is in play
    assert_close_bf16_store(rounded, ref, "rounded to nearest", tol=1e-6)
    with pytest.raises(AssertionError):
        assert_close_bf16_store(truncated, ref, "truncated", tol=1e-6)
    with pytest.raises(AssertionError):
        assert_close_bf16_store(truncated, ref, "truncated", tol=1e-3)


def test_contraction_order_of_the_product_is_the_oracles():
    """decimate.contraction_order packs (cost, mix) into one integer key per edge; on CPU tensors it must order the edges
    exactly as the oracle's lexicographic statement does, for costs that are negative, signed zeros, denormal,
    infinite, NaN or an ulp apart."""
    import torch
    from oracle import decimate_ref as R
    from picassoplus_amd.mesh.pi_modules import decimate as D
    rng = np.random.default_rng(0)
    n = 6000
    vi = np.sort(rng.integers(0, 300, n)).astype(np.int32)
    vj = (vi + rng.integers(1, 50, n)).astype(np.int32)
    k = np.argsort(vi.astype(np.int64) * 1000 + vj, kind="stable")
    vi, vj = vi[k], vj[k]
    special = np.array([0.0, -0.0, 1e-45, -1e-45, 1e-30, -1e-30, -2.5, 2.5, np.nan, np.inf, -np.inf, 1.0, 1.0000001, -1.0], np.float32)
    cost = rng.choice(special, n)
    cost[::7] = rng.normal(size=len(cost[::7])).astype(np.float32)
    for cum in (np.array([100, 200, 300]), np.arange(2, 302, 2)):       # few samples: one key per edge; many: two sorts
        want_perm, want_sample = R.contraction_order(cost, vi, vj, cum)
        perm, sample = D.contraction_order(torch.from_numpy(cost), torch.from_numpy(vi), torch.from_numpy(vj), torch.from_numpy(cum))
        assert np.array_equal(perm.numpy(), want_perm) and np.array_equal(sample.numpy(), want_sample)
    assert np.array_equal(D.edge_mix(torch.from_numpy(vi), torch.from_numpy(vj)).numpy(), R.edge_mix(vi, vj))
