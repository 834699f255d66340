"""facet2vertex backward without a workspace argument (pmesh_f2v_bwd_static): called through the C ABI, its
results must equal pmesh_f2v_bwd's bit for bit (both sum in the same fixed order), on two calls in a row of which
the second has the smaller input (the shared device array still holds the first call's partial sums), and it must
not allocate device memory."""
import numpy as np
import pytest
import torch

from oracle import loops
from picassoplus_amd import _lib, synthetic as S
from picassoplus_amd.mesh import topology
from util import assert_close, dev, mesh_case

pytestmark = pytest.mark.gpu


def _case(cuda, mesh, C, r, seed):
    v, f = mesh_case(mesh)
    rng = np.random.default_rng(seed)
    nv, nf, K = v.shape[0], f.shape[0], 16
    vt_map = np.arange(nv, dtype=np.int32)
    nfc = np.maximum(S.vertex_facet_count(f, vt_map, nv), 1).astype(np.int32)
    a = dict(nv=nv, nf=nf, C=C, r=r, K=K, f=f, nfc=nfc, vt_map=vt_map,
             x=rng.uniform(-1, 1, (nf, C)).astype(np.float32), filt=rng.normal(0, 0.5, (K, C, r)).astype(np.float32),
             coeff=rng.normal(0, 0.5, (nf, K)).astype(np.float32), gout=rng.normal(0, 1, (nv, C * r)).astype(np.float32))
    a["t"] = {k: dev(a[k], cuda) for k in ("x", "filt", "coeff", "gout", "f", "nfc", "vt_map")}
    return a


def _run(a, static):
    t, dv = a["t"], a["t"]["x"].device
    gin = torch.empty(a["nf"], a["C"], device=dv)
    gfilt = torch.empty(a["K"], a["C"], a["r"], device=dv)
    st = torch.cuda.current_stream().cuda_stream
    head = (t["gout"].data_ptr(), t["x"].data_ptr(), t["filt"].data_ptr(), t["coeff"].data_ptr(), t["f"].data_ptr(),
            t["nfc"].data_ptr(), t["vt_map"].data_ptr(), gin.data_ptr(), gfilt.data_ptr())
    dims = (a["nf"], a["nv"], a["nv"], a["C"], a["r"], a["K"], st)
    if static:
        torch.cuda.synchronize()
        # PyTorch's own books, and the device's free memory as the runtime reports it (an allocation made behind
        # PyTorch's back would show there); the array's address is looked up on the first call of the process, so that
        # call runs once before the books are read
        _lib.call("pmesh_f2v_bwd_static", *head, *dims)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0]
        _lib.call("pmesh_f2v_bwd_static", *head, *dims)
        torch.cuda.synchronize()
        assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0]) == before
    else:
        n = _lib.query("pmesh_f2v_bwd_workspace_bytes", a["C"], a["r"], a["K"])
        ws = torch.empty(n, dtype=torch.uint8, device=dv)
        _lib.call("pmesh_f2v_bwd", *head, ws.data_ptr(), n, *dims)
        torch.cuda.synchronize()
    return gin, gfilt


def test_f2v_bwd_static_matches_workspace_entry_point(cuda):
    assert _lib.query("pmesh_f2v_bwd_static_max_bytes") == 8 << 20
    big = _case(cuda, "room_small", 64, 1, 5)        # first call: the larger mesh
    small = _case(cuda, "sphere2", 32, 2, 6)         # second call: fewer facets, other shape, same array
    for a in (big, small):
        print("case f2v_bwd_static", a["nf"], a["C"], a["r"], flush=True)
        gin_s, gfilt_s = _run(a, static=True)
        gin_w, gfilt_w = _run(a, static=False)
        assert torch.equal(gin_s, gin_w) and torch.equal(gfilt_s, gfilt_w)
        ref_gin, ref_gfilt = loops.f2v_bwd(a["gout"], a["x"], a["filt"], a["coeff"], a["f"], a["nfc"], a["vt_map"])
        assert_close(gin_s, ref_gin, "f2v_bwd_static grad_input")
        assert_close(gfilt_s, ref_gfilt, "f2v_bwd_static grad_filter")


def test_f2v_bwd_static_rejects_shapes_beyond_its_array(cuda):
    a = _case(cuda, "tetra", 192, 1, 7)             # 16 * 192 = 3072 > 2048
    with pytest.raises(RuntimeError, match="static array holds"):
        _run(a, static=True)
