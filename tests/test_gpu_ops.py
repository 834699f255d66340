"""Parity of the HIP kernels with the CPU oracle, called through the reference-shaped API.

Reference arithmetic: brute-force loops (oracle/mesh_loops.inc) in float64 for small cases,
the vectorised float64 restatement (oracle/torch_ref.py) for medium ones.  Bar: index arrays
and arg-max indices bit-exact, float32 features and gradients within 1e-5 of max |reference|.
"""
import sys

import numpy as np
import pytest
import torch

from oracle import loops, torch_ref
from picassoplus_amd import synthetic as S
from picassoplus_amd.mesh import topology
from picassoplus_amd.mesh.layers import sph_harm_values
from picassoplus_amd.mesh.pi_modules import (conv3d, mesh_conv3d, mesh_pool3d, mesh_unpool3d, pool3d,
                                             texture, unpool3d)
from util import MEASURED, assert_as_good_as_f32, assert_close, dev, mesh_case, rel_err, strided_vt_map, texture_case

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


# ------------------------------------------------------------------ adjacency
@pytest.mark.parametrize("mesh", ["tetra", "octa", "sphere2", "room_small"])
@pytest.mark.parametrize("strided", [False, True])
def test_vertex_csr_exact(cuda, mesh, strided):
    say("case vertex_csr", mesh, strided)
    v, f = mesh_case(mesh)
    rng = np.random.default_rng(1)
    nv = v.shape[0]
    if strided:
        vt_map, n_rows = strided_vt_map(rng, nv)
        keys = vt_map[f.reshape(-1).astype(np.int64)]
    else:
        vt_map, n_rows = None, nv
        keys = f.reshape(-1).astype(np.int64)
    e = np.arange(keys.shape[0])
    ok = keys >= 0
    order = np.argsort(keys[ok], kind="stable")
    col_ref = e[ok][order].astype(np.int32)
    rowptr_ref = np.concatenate([[0], np.cumsum(np.bincount(keys[ok], minlength=n_rows))]).astype(np.int32)
    rowptr, colidx = topology.vertex_csr(dev(f, cuda), dev(vt_map, cuda) if strided else None, n_rows)
    torch.cuda.synchronize()
    assert np.array_equal(rowptr.cpu().numpy(), rowptr_ref)
    assert np.array_equal(colidx.cpu().numpy()[:col_ref.shape[0]], col_ref)


@pytest.mark.parametrize("spatial", [True, False])
def test_cluster_csr_exact(cuda, spatial):
    say("case cluster_csr", spatial)
    rng = np.random.default_rng(2)
    vt_replace, vt_map, nvo = S.cluster_maps(rng, 5000, spatial=spatial, orphan_frac=0.05)
    vo, _ = torch_ref.cluster_maps(torch.from_numpy(vt_replace), torch.from_numpy(vt_map))
    vo = vo.numpy().astype(np.int64)
    ok = vo >= 0
    ids = np.arange(vo.shape[0])
    order = np.argsort(vo[ok], kind="stable")
    mem_ref = ids[ok][order].astype(np.int32)
    rowptr_ref = np.concatenate([[0], np.cumsum(np.bincount(vo[ok], minlength=nvo))]).astype(np.int32)
    rowptr, members = topology.cluster_csr(dev(vt_replace, cuda), dev(vt_map, cuda), nvo)
    torch.cuda.synchronize()
    assert np.array_equal(rowptr.cpu().numpy(), rowptr_ref)
    assert np.array_equal(members.cpu().numpy()[:mem_ref.shape[0]], mem_ref)


# ------------------------------------------------------------------ vertex2facet
@pytest.mark.parametrize("mesh,C,r", [("tetra", 4, 1), ("octa", 5, 2), ("sphere2", 32, 1), ("sphere3", 64, 1),
                                      ("room_small", 64, 1), ("sphere2", 7, 3), ("torus", 130, 1),
                                      ("octa", 2048, 1), ("sphere2", 96, 1), ("sphere3", 32, 2), ("room_small", 66, 2),
                                      ("sphere2", 128, 2), ("torus", 9, 2)])
def test_v2f_parity(cuda, mesh, C, r):
    say("case v2f", mesh, C, r)
    v, f = mesh_case(mesh)
    rng = np.random.default_rng(10)
    nv, nf = v.shape[0], f.shape[0]
    x = rng.uniform(-1, 1, (nv, C))
    filt = rng.normal(0, 0.5, (3, C, r))
    gout = rng.normal(0, 1, (nf, C * r))
    out_ref = loops.v2f_fwd(x, filt, f)
    gin_ref, gfilt_ref = loops.v2f_bwd(gout, x, filt, f)
    xt = dev(x, cuda, torch.float32).requires_grad_(True)
    ft = dev(filt, cuda, torch.float32).requires_grad_(True)
    out = conv3d.vertex2facet(xt, ft, dev(f, cuda))
    out.backward(dev(gout, cuda, torch.float32))
    torch.cuda.synchronize()
    assert_close(out, out_ref, "v2f out")
    assert_close(xt.grad, gin_ref, "v2f grad_input")
    assert_close(ft.grad, gfilt_ref, "v2f grad_filter")
    # no worse than twice the float32 loops in the reference's summation order
    f32 = np.float32
    gin32, gfilt32 = loops.v2f_bwd(gout.astype(f32), x.astype(f32), filt.astype(f32), f, dtype=f32)
    assert_as_good_as_f32(out, out_ref, loops.v2f_fwd(x.astype(f32), filt.astype(f32), f, dtype=f32), "v2f out")
    assert_as_good_as_f32(xt.grad, gin_ref, gin32, "v2f grad_input")
    assert_as_good_as_f32(ft.grad, gfilt_ref, gfilt32, "v2f grad_filter")


# ------------------------------------------------------------------ texture points from vertex features
@pytest.mark.parametrize("mesh,C,kmax,L", [("tetra", 4, 3, 3), ("octa", 3, 9, 3), ("sphere2", 64, 9, 3), ("fans", 32, 5, 2),
                                           ("room_small", 64, 9, 3), ("room_small", 96, 9, 1), ("fans", 128, 3, 3), ("torus", 130, 4, 5), ("sphere3", 7, 20, None),
                                           ("sphere2", 2048, 2, 0)])
def test_texture_interpolation_parity(cuda, mesh, C, kmax, L):
    say("case texture", mesh, C, kmax, L)
    v, f = mesh_case(mesh)
    rng = np.random.default_rng(12)
    nv, nf = v.shape[0], f.shape[0]
    counts, bary, owner = texture_case(rng, nf, kmax=kmax)
    cum = np.cumsum(counts).astype(np.int32)
    T = int(cum[-1])
    x = rng.uniform(-1, 1, (nv, C))
    g = rng.normal(0, 1, (T, C))
    tex_ref = loops.texture_fwd(x, f, bary, cum)
    gin_ref = loops.texture_bwd(g, nv, f, bary, cum)
    xt = dev(x, cuda, torch.float32).requires_grad_(True)
    bt = dev(bary, cuda, torch.float32)
    res = texture.interpolate(xt, dev(f, cuda), bt, dev(cum, cuda), L)
    tex, coeff = res if L is not None else (res, None)
    tex.backward(dev(g, cuda, torch.float32))
    torch.cuda.synchronize()
    assert_close(tex, tex_ref, "texture features")
    assert_close(xt.grad, gin_ref, "texture grad_input")
    if L is not None:
        assert not coeff.requires_grad
        assert_close(coeff, loops.sph_harm(bt.cpu().numpy().astype(np.float64), L), "texture basis values")
        # the fused basis is the stand-alone kernel's, bit for bit
        assert torch.equal(coeff, sph_harm_values(bt, L))


def test_texture_interpolation_feeds_facet2facet(cuda):
    """Gradient of a facet2facet layer with respect to vertex features through the interpolation, against the
    oracle's composition."""
    say("case texture_chain")
    v, f = mesh_case("sphere3")
    rng = np.random.default_rng(13)
    nv, nf, C, Co, L = v.shape[0], f.shape[0], 16, 32, 3
    counts, bary, owner = texture_case(rng, nf, kmax=4)
    cum = np.cumsum(counts).astype(np.int32)
    x = rng.uniform(-1, 1, (nv, C))
    filt = rng.normal(0, 0.2, (Co, C, (L + 1) ** 2))
    gout = rng.normal(0, 1, (nf, Co))
    T64 = lambda a: torch.from_numpy(np.ascontiguousarray(a))
    sh = torch_ref.sph_harm(T64(bary), L)
    xr = T64(x).requires_grad_(True)
    out_ref = torch_ref.f2f_fwd(torch_ref.texture_fwd(xr, T64(f), T64(bary), T64(cum)), T64(filt), sh, T64(cum))
    (gx_ref,) = torch.autograd.grad(out_ref, xr, T64(gout))
    xt = dev(x, cuda, torch.float32).requires_grad_(True)
    tex, coeff = texture.interpolate(xt, dev(f, cuda), dev(bary, cuda, torch.float32), dev(cum, cuda), L)
    out = conv3d.facet2facet(tex, dev(filt, cuda, torch.float32), coeff, dev(cum, cuda))
    out.backward(dev(gout, cuda, torch.float32))
    torch.cuda.synchronize()
    assert_close(out, out_ref.detach().numpy(), "chain out")
    assert_close(xt.grad, gx_ref.numpy(), "chain grad_input")


def test_texture_interpolation_rejects_bad_totals(cuda):
    say("case texture_bad_totals")
    x = torch.zeros(4, 8, device=cuda)
    face = torch.tensor([[0, 1, 2], [1, 2, 3]], dtype=torch.int32, device=cuda)
    bary = torch.full((5, 3), 1 / 3, device=cuda)
    with pytest.raises(RuntimeError, match="running total"):
        texture.interpolate(x, face, bary, torch.tensor([2, 4], dtype=torch.int32, device=cuda))
    with pytest.raises(RuntimeError, match="running total"):
        texture.interpolate(x, face, bary, torch.tensor([6, 5], dtype=torch.int32, device=cuda))
    with pytest.raises(RuntimeError, match="one running total per facet"):
        texture.interpolate(x, face, bary, torch.tensor([5], dtype=torch.int32, device=cuda))
    empty = texture.interpolate(x, face, bary[:0], torch.zeros(2, dtype=torch.int32, device=cuda))
    assert empty[0].shape == (0, 8) and empty[1].shape == (0, 16)


# ------------------------------------------------------------------ facet2vertex
@pytest.mark.parametrize("mesh,C,r,K,strided", [("tetra", 4, 1, 16, False), ("octa", 6, 2, 9, True),
                                                ("sphere2", 32, 1, 16, False), ("sphere3", 64, 1, 16, True),
                                                ("room_small", 64, 1, 16, False), ("torus", 20, 1, 36, False),
                                                ("sphere2", 5, 3, 4, True), ("sphere2", 128, 1, 16, False),
                                                ("sphere3", 48, 2, 16, True), ("sphere3", 96, 1, 16, False),
                                                ("room_small", 40, 2, 9, True), ("sphere2", 36, 2, 16, False),
                                                ("sphere2", 160, 1, 12, True), ("sphere2", 64, 2, 16, False),
                                                ("fans", 64, 1, 16, False), ("fans", 40, 1, 16, True),
                                                ("sphere3", 200, 1, 16, True), ("sphere2", 12, 3, 16, False),
                                                ("room_small", 128, 2, 16, True), ("sphere3", 33, 1, 16, False),
                                                ("sphere3", 64, 1, 25, False), ("room_small", 32, 2, 36, True)])
@pytest.mark.parametrize("path", ["default", "valu", "fp32mfma"])
def test_f2v_parity(cuda, native_options, mesh, C, r, K, strided, path):
    """default: matrix-core kernels where they apply (at least 32 output channels; 16 coefficients, or from 9 on as
    zero-padded blocks of 16), the forward's filter combination as two-piece fp16 products; fp32mfma: the same kernels
    with that product on the fp32 matrix instruction; valu: the vector-ALU kernels for every shape."""
    say("case f2v", mesh, C, r, K, strided, path)
    native_options(PMESH_F2V_VALU="1" if path == "valu" else "0", PMESH_F2V_FP32MFMA="1" if path == "fp32mfma" else "0")
    v, f = mesh_case(mesh)
    rng = np.random.default_rng(11)
    nv, nf = v.shape[0], f.shape[0]
    if strided:
        vt_map, nvo = strided_vt_map(rng, nv)
    else:
        vt_map, nvo = np.arange(nv, dtype=np.int32), nv
    nfc = S.vertex_facet_count(f, vt_map, nvo)
    x = rng.uniform(-1, 1, (nf, C))
    filt = rng.normal(0, 0.5, (K, C, r))
    coeff = rng.normal(0, 0.5, (nf, K))
    gout = rng.normal(0, 1, (nvo, C * r))
    out_ref = loops.f2v_fwd(x, filt, coeff, f, np.maximum(nfc, 1), vt_map)
    gin_ref, gfilt_ref = loops.f2v_bwd(gout, x, filt, coeff, f, np.maximum(nfc, 1), vt_map)
    xt = dev(x, cuda, torch.float32).requires_grad_(True)
    ft = dev(filt, cuda, torch.float32).requires_grad_(True)
    out = conv3d.facet2vertex(xt, ft, dev(coeff, cuda, torch.float32), dev(f, cuda),
                              dev(np.maximum(nfc, 1), cuda), dev(vt_map, cuda))
    out.backward(dev(gout, cuda, torch.float32))
    torch.cuda.synchronize()
    assert_close(out, out_ref, "f2v out")
    assert_close(xt.grad, gin_ref, "f2v grad_input")
    assert_close(ft.grad, gfilt_ref, "f2v grad_filter")
    f32 = np.float32
    a32 = (x.astype(f32), filt.astype(f32), coeff.astype(f32), f, np.maximum(nfc, 1), vt_map)
    gin32, gfilt32 = loops.f2v_bwd(gout.astype(f32), *a32, dtype=f32)
    assert_as_good_as_f32(out, out_ref, loops.f2v_fwd(*a32, dtype=f32), "f2v out")
    assert_as_good_as_f32(xt.grad, gin_ref, gin32, "f2v grad_input")
    assert_as_good_as_f32(ft.grad, gfilt_ref, gfilt32, "f2v grad_filter")


@pytest.mark.parametrize("cscale,fscale", [(1e-12, 1e6), (1e12, 1e-9), (3e-5, 7e4)])
def test_f2v_coefficients_and_filters_far_from_one(cuda, cscale, fscale):
    """The two-piece fp16 products bring coefficients and filter columns into fp16's range by powers of two: inputs
    twelve orders of magnitude above or below one come out to the same 1e-5 (no overflow to infinity, no loss to
    fp16's subnormal range), and an all-zero coefficient row stays an exact zero."""
    say("case f2v magnitudes", cscale, fscale)
    v, f = mesh_case("sphere3")
    rng = np.random.default_rng(15)
    nv, nf, C, K = v.shape[0], f.shape[0], 64, 16
    vt_map = np.arange(nv, dtype=np.int32)
    nfc = np.maximum(S.vertex_facet_count(f, vt_map, nv), 1)
    r32 = lambda a: a.astype(np.float32).astype(np.float64)
    x = r32(rng.uniform(-1, 1, (nf, C)))
    filt = r32(rng.normal(0, 0.5, (K, C, 1)) * fscale)
    coeff = r32(rng.normal(0, 0.5, (nf, K)) * cscale)
    coeff[::7] = 0.0
    gout = r32(rng.normal(0, 1, (nv, C)))
    out_ref = loops.f2v_fwd(x, filt, coeff, f, nfc, vt_map)
    gin_ref, gfilt_ref = loops.f2v_bwd(gout, x, filt, coeff, f, nfc, vt_map)
    xt = dev(x, cuda, torch.float32).requires_grad_(True)
    ft = dev(filt, cuda, torch.float32).requires_grad_(True)
    out = conv3d.facet2vertex(xt, ft, dev(coeff, cuda, torch.float32), dev(f, cuda), dev(nfc, cuda), dev(vt_map, cuda))
    out.backward(dev(gout, cuda, torch.float32))
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(xt.grad).all()) and bool(torch.isfinite(ft.grad).all())
    assert_close(out, out_ref, "f2v out, magnitudes far from one")
    assert_close(xt.grad, gin_ref, "f2v grad_input, magnitudes far from one")
    assert_close(ft.grad, gfilt_ref, "f2v grad_filter, magnitudes far from one")


@pytest.mark.parametrize("path", ["default", "fp32mfma"])
def test_f2v_channels_of_very_different_size(cuda, native_options, path):
    """Filter columns and feature channels nine orders of magnitude apart: every channel is held to 1e-5 of ITS OWN
    largest value (the matrix-core kernels scale each filter column and each channel of the second product by its own
    power of two; one scale for all of them would leave the small channels with a few bits)."""
    say("case f2v channel scales", path)
    native_options(PMESH_F2V_FP32MFMA="1" if path == "fp32mfma" else "0")
    v, f = mesh_case("sphere3")
    rng = np.random.default_rng(14)
    nv, nf, C, K = v.shape[0], f.shape[0], 64, 16
    vt_map = np.arange(nv, dtype=np.int32)
    nfc = np.maximum(S.vertex_facet_count(f, vt_map, nv), 1)
    col = 10.0 ** rng.uniform(-6, 3, C)
    x = rng.uniform(-1, 1, (nf, C)) * 10.0 ** rng.uniform(-3, 3, C)
    filt = rng.normal(0, 0.5, (K, C, 1)) * col[None, :, None]
    coeff = rng.normal(0, 0.5, (nf, K))
    gout = rng.normal(0, 1, (nv, C)) * 10.0 ** rng.uniform(-3, 3, C)
    xt = dev(x, cuda, torch.float32).requires_grad_(True)
    ft = dev(filt, cuda, torch.float32).requires_grad_(True)
    out = conv3d.facet2vertex(xt, ft, dev(coeff, cuda, torch.float32), dev(f, cuda), dev(nfc, cuda), dev(vt_map, cuda))
    out.backward(dev(gout, cuda, torch.float32))
    torch.cuda.synchronize()
    # the float32 inputs are the oracle's inputs rounded: compare against the oracle on the rounded inputs
    r32 = lambda a: a.astype(np.float32).astype(np.float64)
    out_ref = loops.f2v_fwd(r32(x), r32(filt), r32(coeff), f, nfc, vt_map)
    gin_ref, gfilt_ref = loops.f2v_bwd(r32(gout), r32(x), r32(filt), r32(coeff), f, nfc, vt_map)
    for name, got, ref in (("out", out, out_ref), ("grad_input", xt.grad, gin_ref), ("grad_filter", ft.grad[:, :, 0], gfilt_ref[:, :, 0])):
        got = got.detach().cpu().numpy().astype(np.float64)
        worst = max(np.abs(got[:, c] - ref[:, c]).max() / np.abs(ref[:, c]).max() for c in range(C))
        MEASURED.append(("f2v %s, worst channel relative to its own maximum [%s]" % (name, path), worst, 1e-5))
        assert worst <= 1e-5, (name, worst)


def test_f2v_unit_count_is_plain_scatter(cuda):
    """nf_count = 1 and a one-hot coeff reduce facet2vertex to a scatter-add of filt[k0]*x."""
    say("case f2v one-hot")
    v, f = mesh_case("sphere2")
    rng = np.random.default_rng(12)
    nv, nf, C, K = v.shape[0], f.shape[0], 8, 16
    x = rng.uniform(-1, 1, (nf, C)).astype(np.float32)
    filt = rng.normal(0, 1, (K, C, 1)).astype(np.float32)
    coeff = np.zeros((nf, K), np.float32)
    coeff[:, 3] = 1
    ref = np.zeros((nv, C))
    np.add.at(ref, f.reshape(-1), np.repeat(x.astype(np.float64) * filt[3, :, 0], 3, axis=0))
    out = mesh_conv3d.facet2vertex_forward(dev(x, cuda), dev(filt, cuda), dev(coeff, cuda), dev(f, cuda),
                                           dev(np.ones(nv, np.int32), cuda), dev(np.arange(nv, dtype=np.int32), cuda))
    torch.cuda.synchronize()
    assert_close(out, ref, "f2v scatter form")


# ------------------------------------------------------------------ facet2facet
@pytest.mark.parametrize("nf,Cin,Cout,F,kmax", [(10, 3, 8, 16, 3), (100, 3, 32, 16, 5), (200, 64, 64, 16, 9),
                                                (333, 16, 96, 16, 4), (70, 5, 7, 9, 3), (65, 4, 6, 36, 2),
                                                (64, 3, 5, 50, 2), (129, 130, 64, 4, 3), (50, 8, 8, 1, 2),
                                                (300, 8, 40, 16, 14), (1000, 64, 64, 16, 9), (130, 4, 130, 16, 20),
                                                (50, 1, 8, 16, 3), (77, 2, 33, 16, 12),
                                                (300, 128, 128, 16, 9), (260, 256, 256, 16, 9), (150, 128, 256, 16, 6),
                                                (90, 256, 128, 16, 4), (200, 32, 32, 16, 9)])
@pytest.mark.parametrize("path", ["default", "generic", "bf16x3", "half"])
def test_f2f_parity(cuda, native_options, nf, Cin, Cout, F, kmax, path):
    """``generic`` forces the shape-generic kernels (fp32 matrix instruction) and ``bf16x3`` the three-piece bf16
    kernels, also where the two-piece fp16 kernels (the default, 16 coefficients per block) apply; ``half`` their
    half-precision variant (one fp16 piece per operand, fp32 accumulation), held to 1e-3 of the largest reference
    value instead of 1e-5."""
    say("case f2f", nf, Cin, Cout, F, kmax, path)
    # other coefficient counts than 16 run as blocks of 16 (zero padded) through whichever split kernels are selected;
    # ``generic`` takes them as they are
    native_options(PMESH_F2F_HALF="1" if path == "half" else "0", PMESH_F2F_GENERIC="1" if path == "generic" else "0",
                   PMESH_F2F_BF16X3="1" if path == "bf16x3" else "0")
    rng = np.random.default_rng(13)
    counts, bary, owner = texture_case(rng, nf, kmax)
    cum = np.cumsum(counts).astype(np.int32)
    T = int(counts.sum()) + (3 if nf % 2 else 0)       # some cases carry texture rows that belong to no facet
    tex = rng.uniform(-1, 1, (T, Cin))
    sh = rng.normal(0, 0.5, (T, F))
    filt = rng.normal(0, 0.3, (Cout, Cin, F))
    gout = rng.normal(0, 1, (nf, Cout))
    out_ref = loops.f2f_fwd(tex, filt, sh, cum)
    gin_ref, gfilt_ref = loops.f2f_bwd(gout, tex, filt, sh, cum)
    tt = dev(tex, cuda, torch.float32).requires_grad_(True)
    ft = dev(filt, cuda, torch.float32).requires_grad_(True)
    out = conv3d.facet2facet(tt, ft, dev(sh, cuda, torch.float32), dev(cum, cuda))
    out.backward(dev(gout, cuda, torch.float32))
    torch.cuda.synchronize()
    tol = 1e-3 if path == "half" else 1e-5
    e = [assert_close(out, out_ref, "f2f out", tol), assert_close(tt.grad, gin_ref, "f2f grad_texture", tol),
         assert_close(ft.grad, gfilt_ref, "f2f grad_filter", tol)]
    if path == "half" and Cin > 4 and Cin % 4 == 0 and Cout % 8 == 0:
        assert max(e) > 2e-6, "the half-precision variant did not run"         # it is not the full-precision result
    if path != "half":
        f32 = np.float32
        a32 = (tex.astype(f32), filt.astype(f32), sh.astype(f32), cum)
        gin32, gfilt32 = loops.f2f_bwd(gout.astype(f32), *a32, dtype=f32)
        # the production path is held to the criterion; the cross-check paths only report their figures
        k = 3.0 if path == "default" else None
        e_o = assert_as_good_as_f32(out, out_ref, loops.f2f_fwd(*a32, dtype=f32), "f2f out", k)
        e_t = assert_as_good_as_f32(tt.grad, gin_ref, gin32, "f2f grad_texture", k)
        e_w = assert_as_good_as_f32(ft.grad, gfilt_ref, gfilt32, "f2f grad_filter", k)
        say("  errors (build, float32 oracle): out %.2e %.2e  grad_texture %.2e %.2e  grad_filter %.2e %.2e" % (e_o + e_t + e_w))


@pytest.mark.parametrize("nf,Cin,Cout,F,kmax", [(200, 64, 64, 16, 9), (333, 16, 96, 16, 4), (300, 8, 40, 16, 14),
                                                (100, 3, 32, 16, 5), (70, 5, 7, 9, 3), (260, 128, 256, 16, 6)])
@pytest.mark.parametrize("relu", [True, False])
def test_f2f_fused_tail_parity(cuda, nf, Cin, Cout, F, kmax, relu):
    """facet2facet with bias and ReLU on the convolution's store (the first steps of F2FConv3d's tail,
    picasso/mesh/layers.py:59-63) against the oracle's composition in float64, gradients included; the shapes cover the
    fp16 kernels that fuse the tail, with and without the bit form of the mask (Cout % 32), and the kernels that run
    the tail as a second pass (narrow, generic).  Inference form: scale and shift of a frozen batch norm as well."""
    say("case f2f fused tail", nf, Cin, Cout, F, kmax, relu)
    rng = np.random.default_rng(31)
    counts, bary, owner = texture_case(rng, nf, kmax)
    cum = np.cumsum(counts).astype(np.int32)
    T = int(counts.sum())
    tex = rng.uniform(-1, 1, (T, Cin))
    sh = rng.normal(0, 0.5, (T, F))
    filt = rng.normal(0, 0.3, (Cout, Cin, F))
    bias = rng.normal(0, 0.5, Cout)
    gout = rng.normal(0, 1, (nf, Cout))
    conv = loops.f2f_fwd(tex, filt, sh, cum)
    z = conv + bias
    # keep the comparison away from the kink: values within the build's error of zero may land on either side
    z_safe = np.abs(z) > 1e-4 * np.abs(conv).max()
    out_ref = np.maximum(z, 0) if relu else z
    tt = dev(tex, cuda, torch.float32).requires_grad_(True)
    ft = dev(filt, cuda, torch.float32).requires_grad_(True)
    bt = dev(bias, cuda, torch.float32).requires_grad_(True)
    sht, cumt = dev(sh, cuda, torch.float32), dev(cum, cuda)
    out = conv3d.facet2facet_bias_act(tt, ft, bt, sht, cumt, relu)
    g = gout * z_safe                                          # no gradient through entries too close to the kink
    gin_ref, gfilt_ref = loops.f2f_bwd(g * (z > 0) if relu else g, tex, filt, sh, cum)
    out.backward(dev(g, cuda, torch.float32))
    torch.cuda.synchronize()
    o = out.detach().cpu().numpy()
    assert np.abs(o - out_ref).max() <= 1e-5 * np.abs(conv).max(), "fused out"
    if relu:
        assert np.array_equal(o[z_safe] > 0, z[z_safe] > 0)
    assert_close(tt.grad, gin_ref, "fused grad_texture")
    assert_close(ft.grad, gfilt_ref, "fused grad_filter")
    assert_close(bt.grad, (g * (z > 0) if relu else g).sum(0), "fused grad_bias")
    # the same values as the two-step path of the module
    two = torch.relu(conv3d.facet2facet(tt.detach(), ft.detach(), sht, cumt) + bt.detach()) if relu else \
        conv3d.facet2facet(tt.detach(), ft.detach(), sht, cumt) + bt.detach()
    assert float((out.detach() - two).abs().max()) <= 3e-7 * np.abs(conv).max(), "fused and two-step results differ"
    # inference form with a frozen batch norm
    scale, shift = rng.uniform(0.5, 2, Cout), rng.normal(0, 1, Cout)
    y = mesh_conv3d.facet2facet_forward_act(tt.detach(), ft.detach(), sht, cumt, bt.detach(), relu,
                                            dev(scale, cuda, torch.float32), dev(shift, cuda, torch.float32))
    want = out_ref * scale + shift
    assert np.abs(y.cpu().numpy() - want).max() <= 1e-5 * max(np.abs(want).max(), np.abs(conv).max() * scale.max())
    if Cout % 32 == 0 and relu:
        y2, bits = mesh_conv3d.facet2facet_forward_act(tt.detach(), ft.detach(), sht, cumt, bt.detach(), True, with_bits=True)
        assert torch.equal(y2, out.detach())
        b = bits.cpu().numpy().view(np.uint32)
        mask = ((b[:, :, None] >> np.arange(32, dtype=np.uint32)) & 1).reshape(nf, Cout).astype(bool)
        assert np.array_equal(mask, o > 0)


@pytest.mark.parametrize("case", ["late_channels", "late_points", "growing_facets"])
def test_f2f_wide_dynamic_range(cuda, case):
    """The fp16 kernels choose power-of-two operand scales from what they have seen so far and must recover when
    later data is larger by orders of magnitude: channels past the first eight (forward: first bound exceeded,
    workgroup redone with exact maxima), later texture points / their SH rows, and facets whose magnitudes grow
    along the sorted facet list (filter gradient: operand split again with a new scale; passes accumulated
    several times when the accumulator scale no longer fits)."""
    say("case f2f dynamic range", case)
    rng = np.random.default_rng(99)
    nf, Cin, Cout = 700, 32, 64
    counts, bary, owner = texture_case(rng, nf, 9)
    cum = np.cumsum(counts).astype(np.int32)
    T = int(counts.sum())
    tex = rng.uniform(-1, 1, (T, Cin))
    sh = rng.normal(0, 0.5, (T, 16))
    filt = rng.normal(0, 0.3, (Cout, Cin, 16))
    gout = rng.normal(0, 1, (nf, Cout))
    first = np.concatenate([[0], cum[:-1]])
    local = np.arange(T) - first[owner]                      # index of a point inside its facet
    if case == "late_channels":
        tex[:, 8:] *= 3000.0
        tex[owner % 3 == 0, 20] *= 50.0
    elif case == "late_points":
        tex[local >= 4] *= 500.0
        sh[local >= 5] *= 200.0
    else:
        mag = 10.0 ** (counts[owner] * 1.2 - 3)              # 1e-3 .. 1e8 with the number of points
        tex *= mag[:, None]
        gout *= (10.0 ** (counts * 0.9 - 2))[:, None]
    out_ref = loops.f2f_fwd(tex, filt, sh, cum)
    gin_ref, gfilt_ref = loops.f2f_bwd(gout, tex, filt, sh, cum)
    tt = dev(tex, cuda, torch.float32).requires_grad_(True)
    ft = dev(filt, cuda, torch.float32).requires_grad_(True)
    out = conv3d.facet2facet(tt, ft, dev(sh, cuda, torch.float32), dev(cum, cuda))
    out.backward(dev(gout, cuda, torch.float32))
    torch.cuda.synchronize()
    assert_close(out, out_ref, "f2f out")
    assert_close(tt.grad, gin_ref, "f2f grad_texture")
    assert_close(ft.grad, gfilt_ref, "f2f grad_filter")


@pytest.mark.parametrize("case", ["zero_grad_rows", "relu_sparse", "all_zero", "zero_filter"])
def test_f2f_sparse_and_zero_data(cuda, case):
    """Data a trained network really produces: facets without a label send all-zero gradient rows, a ReLU in front
    leaves half of the texture features zero and whole facets dark, and a freshly zeroed filter or an all-zero
    gradient must give exact zeros, never a NaN from a scale of an empty maximum."""
    say("case f2f sparse", case)
    rng = np.random.default_rng(123)
    nf, Cin, Cout = 1500, 32, 64
    counts, bary, owner = texture_case(rng, nf, 7)
    cum = np.cumsum(counts).astype(np.int32)
    T = int(counts.sum())
    tex = rng.normal(0, 1, (T, Cin))
    sh = rng.normal(0, 0.5, (T, 16))
    filt = rng.normal(0, 0.3, (Cout, Cin, 16))
    gout = rng.normal(0, 1, (nf, Cout))
    if case == "zero_grad_rows":
        gout[rng.random(nf) < 0.7] = 0.0
        gout[:200] = 0.0                                     # whole tiles of facets without a gradient
    elif case == "relu_sparse":
        tex = np.maximum(tex, 0.0)
        tex[np.isin(owner, np.nonzero(rng.random(nf) < 0.3)[0])] = 0.0
        gout = np.where(rng.random((nf, Cout)) < 0.5, gout, 0.0)
    elif case == "all_zero":
        gout[:] = 0.0
        tex[:] = 0.0
    else:
        filt[:] = 0.0
    out_ref = loops.f2f_fwd(tex, filt, sh, cum)
    gin_ref, gfilt_ref = loops.f2f_bwd(gout, tex, filt, sh, cum)
    tt = dev(tex, cuda, torch.float32).requires_grad_(True)
    ft = dev(filt, cuda, torch.float32).requires_grad_(True)
    out = conv3d.facet2facet(tt, ft, dev(sh, cuda, torch.float32), dev(cum, cuda))
    out.backward(dev(gout, cuda, torch.float32))
    torch.cuda.synchronize()
    for name, got, ref in (("out", out, out_ref), ("grad_texture", tt.grad, gin_ref), ("grad_filter", ft.grad, gfilt_ref)):
        assert bool(torch.isfinite(got).all()), name
        if np.abs(ref).max() == 0.0:
            assert float(got.detach().abs().max()) == 0.0, name
        else:
            assert_close(got, ref, "f2f " + name)


def test_f2f_without_facet_order(cuda):
    """The facet order is optional at the C ABI (NULL): same results for the forward and the texture gradient
    (to an ulp), the same filter gradient up to summation order."""
    from picassoplus_amd import _lib
    from picassoplus_amd.mesh import topology
    say("case f2f without facet order")
    rng = np.random.default_rng(55)
    nf, Cin, Cout = 900, 24, 40
    counts, bary, _ = texture_case(rng, nf, 11)
    T = int(counts.sum())
    tex = dev(rng.uniform(-1, 1, (T, Cin)), cuda, torch.float32)
    sh = dev(rng.normal(0, 0.5, (T, 16)), cuda, torch.float32)
    w = dev(rng.normal(0, 0.3, (Cout, Cin, 16)), cuda, torch.float32)
    g = dev(rng.normal(0, 1, (nf, Cout)), cuda, torch.float32)
    cum = torch.cumsum(dev(counts, cuda), 0, dtype=torch.int32)
    order = topology.facet_order(cum, T)
    st = torch.cuda.current_stream().cuda_stream
    nfw = _lib.query("pmesh_f2f_fwd_workspace_bytes", Cin, Cout, 16)
    nbw = _lib.query("pmesh_f2f_bwd_workspace_bytes", Cin, Cout, 16)
    ws = torch.empty(max(nfw, nbw), dtype=torch.uint8, device=cuda)
    res = []
    for o in (order.data_ptr(), None):
        out = torch.empty(nf, Cout, device=cuda)
        gtex = torch.empty(T, Cin, device=cuda)
        gw = torch.empty(Cout, Cin, 16, device=cuda)
        _lib.call("pmesh_f2f_fwd", tex.data_ptr(), w.data_ptr(), sh.data_ptr(), cum.data_ptr(), o, out.data_ptr(),
                  ws.data_ptr(), nfw, T, nf, Cin, Cout, 16, st)
        _lib.call("pmesh_f2f_bwd", g.data_ptr(), tex.data_ptr(), w.data_ptr(), sh.data_ptr(), cum.data_ptr(), o,
                  gtex.data_ptr(), gw.data_ptr(), ws.data_ptr(), nbw, T, nf, Cin, Cout, 16, st)
        torch.cuda.synchronize()
        res.append((out, gtex, gw))
    (o1, t1, w1), (o2, t2, w2) = res
    assert float((o1 - o2).abs().max()) <= 2e-7 * float(o1.abs().max())
    assert float((t1 - t2).abs().max()) <= 2e-7 * float(t1.abs().max())
    assert float((w1 - w2).abs().max()) <= 1e-5 * float(w1.abs().max())


@pytest.mark.parametrize("nf,Cin,Cout", [(900, 24, 40), (257, 64, 64), (130, 8, 128)])
def test_f2f_texture_gradient_added_in_place(cuda, nf, Cin, Cout):
    """pmesh_f2f_bwd_texture_onto adds the texture gradient to what the array holds -- rows that belong to no facet stay
    as they are -- and gives the plain entry point's result on top of it; the coefficient blocks of another degree are
    cut once per tensor and cut again when the tensor's contents change."""
    from picassoplus_amd import _lib
    say("case f2f texture gradient in place", nf, Cin, Cout)
    rng = np.random.default_rng(56)
    counts, bary, _ = texture_case(rng, nf, 9)
    T = int(counts.sum()) + 5                              # five rows that belong to no facet
    sh = dev(rng.normal(0, 0.5, (T, 16)), cuda, torch.float32)
    w = dev(rng.normal(0, 0.3, (Cout, Cin, 16)), cuda, torch.float32)
    g = dev(rng.normal(0, 1, (nf, Cout)), cuda, torch.float32)
    cum = torch.cumsum(dev(counts, cuda), 0, dtype=torch.int32)
    order = topology.facet_order(cum, T)
    st = torch.cuda.current_stream().cuda_stream
    nbw = _lib.query("pmesh_f2f_bwd_workspace_bytes", Cin, Cout, 16)
    ws = torch.empty(nbw, dtype=torch.uint8, device=cuda)
    assert _lib.query("pmesh_f2f_bwd_texture_onto_supported", g.data_ptr(), w.data_ptr(), sh.data_ptr(), Cout, 16) == 1
    plain = torch.empty(T, Cin, device=cuda)
    _lib.call("pmesh_f2f_bwd_texture", g.data_ptr(), w.data_ptr(), sh.data_ptr(), cum.data_ptr(), order.data_ptr(),
              plain.data_ptr(), ws.data_ptr(), nbw, T, nf, Cin, Cout, 16, st)
    base = torch.randn(T, Cin, device=cuda)
    onto = base.clone()
    _lib.call("pmesh_f2f_bwd_texture_onto", g.data_ptr(), w.data_ptr(), sh.data_ptr(), cum.data_ptr(), order.data_ptr(),
              onto.data_ptr(), ws.data_ptr(), nbw, T, nf, Cin, Cout, 16, st)
    torch.cuda.synchronize()
    assert torch.equal(plain[-5:], torch.zeros(5, Cin, device=cuda)) and torch.equal(onto[-5:], base[-5:])
    assert float((onto - (base + plain)).abs().max()) <= 2e-7 * float((base.abs() + plain.abs()).max())
    # other degrees: the cached coefficient blocks follow the tensor's contents
    sh25 = dev(rng.normal(0, 0.5, (T, 25)), cuda, torch.float32)
    b1 = topology.coefficient_blocks(sh25)
    assert topology.coefficient_blocks(sh25) is b1 and len(b1) == 2 and tuple(b1[1].shape) == (T, 16)
    assert torch.equal(b1[0], sh25[:, :16]) and torch.equal(b1[1][:, :9], sh25[:, 16:]) and not b1[1][:, 9:].any()
    sh25.mul_(2.0)
    b2 = topology.coefficient_blocks(sh25)
    assert b2 is not b1 and torch.equal(b2[0], sh25[:, :16])


def test_f2f_shape_sweep(cuda):
    """Seeded sweep over channel counts, facet counts and point counts around the tile sizes of the
    16-coefficient kernels (32-facet wavefront tiles, 4/8/16-channel groups, 64-channel blocks)."""
    rng = np.random.default_rng(77)
    cins = [4, 8, 12, 20, 36, 64, 68, 132]
    couts = [8, 16, 24, 40, 64, 72, 128, 5]
    nfs = [1, 31, 32, 33, 255, 257, 700]
    kmaxs = [1, 2, 4, 5, 9, 13]
    for it in range(28):
        Cin, Cout = cins[it % len(cins)], couts[(it * 3 + 1) % len(couts)]
        nf, kmax = nfs[(it * 5 + 2) % len(nfs)], kmaxs[(it * 7 + 3) % len(kmaxs)]
        say("case f2f sweep", it, nf, Cin, Cout, kmax)
        counts, bary, owner = texture_case(rng, nf, kmax, empty_frac=0.1 if nf > 1 else 0.0)
        cum = np.cumsum(counts).astype(np.int32)
        T = int(counts.sum()) + (it % 3)
        tex = rng.uniform(-1, 1, (T, Cin))
        sh = rng.normal(0, 0.5, (T, 16))
        filt = rng.normal(0, 0.3, (Cout, Cin, 16))
        gout = rng.normal(0, 1, (nf, Cout))
        out_ref = loops.f2f_fwd(tex, filt, sh, cum)
        gin_ref, gfilt_ref = loops.f2f_bwd(gout, tex, filt, sh, cum)
        tt = dev(tex, cuda, torch.float32).requires_grad_(True)
        ft = dev(filt, cuda, torch.float32).requires_grad_(True)
        out = conv3d.facet2facet(tt, ft, dev(sh, cuda, torch.float32), dev(cum, cuda))
        out.backward(dev(gout, cuda, torch.float32))
        torch.cuda.synchronize()
        tag = " (sweep %d: nf=%d Cin=%d Cout=%d kmax=%d)" % (it, nf, Cin, Cout, kmax)
        assert_close(out, out_ref, "f2f out" + tag)
        assert_close(tt.grad, gin_ref, "f2f grad_texture" + tag)
        assert_close(ft.grad, gfilt_ref, "f2f grad_filter" + tag)


# ------------------------------------------------------------------ pooling
@pytest.mark.parametrize("nv,C,spatial,orphans", [(50, 4, True, 0.0), (3000, 128, True, 0.05), (3000, 5, False, 0.1),
                                                  (777, 64, False, 0.0), (100, 1100, True, 0.0)])
def test_pool_unpool_parity(cuda, nv, C, spatial, orphans):
    say("case pool", nv, C, spatial, orphans)
    rng = np.random.default_rng(14)
    vt_replace, vt_map, nvo = S.cluster_maps(rng, nv, spatial=spatial, orphan_frac=orphans)
    x = rng.normal(0, 1, (nv, C)).astype(np.float32)
    gout = rng.normal(0, 1, (nvo, C)).astype(np.float32)
    gfine = rng.normal(0, 1, (nv, C)).astype(np.float32)
    vr, vm = dev(vt_replace, cuda), dev(vt_map, cuda)
    vt_out = torch.zeros(nvo, 3, device=cuda)

    # max pool: value and arg-max bit-exact (inputs are float32 on both sides)
    out_ref, idx_ref = loops.maxpool_fwd(x, vt_replace, vt_map, nvo, dtype=np.float32)
    xt = dev(x, cuda).requires_grad_(True)
    out, idx = mesh_pool3d.max_forward(xt.detach(), vr, vm, vt_out)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), out_ref)
    assert np.array_equal(idx.cpu().numpy(), idx_ref)
    y = pool3d.maxPool(xt, vr, vm, vt_out)
    y.backward(dev(gout, cuda))
    gin_ref = loops.maxpool_bwd(gout, nv, idx_ref, dtype=np.float32)
    torch.cuda.synchronize()
    assert np.array_equal(xt.grad.cpu().numpy(), gin_ref)
    gin_scatter = mesh_pool3d.max_backward(dev(gout, cuda), xt.detach(), idx)
    torch.cuda.synchronize()
    assert np.array_equal(gin_scatter.cpu().numpy(), gin_ref)

    # avg pool
    xt = dev(x, cuda).requires_grad_(True)
    y = pool3d.avgPool(xt, vr, vm, vt_out)
    y.backward(dev(gout, cuda))
    torch.cuda.synchronize()
    assert_close(y, loops.avgpool_fwd(x, vt_replace, vt_map, nvo), "avg out")
    assert_close(xt.grad, loops.avgpool_bwd(gout, vt_replace, vt_map), "avg grad")

    # unpool (copy: exact) and its backward
    ct = dev(gout, cuda).requires_grad_(True)
    up = unpool3d.interpolate(ct, vr, vm)
    up.backward(dev(gfine, cuda))
    torch.cuda.synchronize()
    assert np.array_equal(up.detach().cpu().numpy(), loops.unpool_fwd(gout, vt_replace, vt_map, dtype=np.float32))
    assert_close(ct.grad, loops.unpool_bwd(gfine, nvo, vt_replace, vt_map), "unpool grad")


def test_max_pool_tie_rule_and_empty_rows(cuda):
    """Equal values: the smallest vertex id wins.  Output rows past the last cluster stay 0 / index 0."""
    say("case pool ties")
    vt_replace = np.array([0, 2, -1, -1, 0, -6, 1], np.int32)   # clusters {0}, {1,2,3}, {4}, {6,5}
    vt_map = np.array([0, 1, -1, -1, 2, -1, 3], np.int32)
    x = np.array([[1, 5], [7, 2], [7, 9], [3, 9], [-4, -4], [0.5, 6], [0.5, -1]], np.float32)
    out, idx = mesh_pool3d.max_forward(dev(x, cuda), dev(vt_replace, cuda), dev(vt_map, cuda),
                                       torch.zeros(6, 3, device=cuda))
    torch.cuda.synchronize()
    assert out.cpu().tolist() == [[1, 5], [7, 9], [-4, -4], [0.5, 6], [0, 0], [0, 0]]
    assert idx.cpu().tolist() == [[0, 0], [1, 2], [4, 4], [5, 5], [0, 0], [0, 0]]


# ------------------------------------------------------------------ spherical harmonics
@pytest.mark.parametrize("L", [0, 1, 2, 3, 4, 5])
def test_sph_harm_parity(cuda, L):
    say("case sph_harm", L)
    rng = np.random.default_rng(15)
    xyz = rng.normal(0, 1, (2000, 3)) * rng.uniform(1e-3, 1e3, (2000, 1))
    xyz[:7] = [[0, 0, 0], [1, 0, 0], [0, 1, 0], [0, 0, 1], [-1, 0, 0], [0, -1, 0], [0, 0, -1]]
    xyz32 = xyz.astype(np.float32)
    ref = loops.sph_harm(xyz32.astype(np.float64), L)
    out = sph_harm_values(dev(xyz32, cuda), L)
    torch.cuda.synchronize()
    assert_close(out, ref, "sph_harm L=%d" % L)


# ------------------------------------------------------------------ determinism
def test_bitwise_reproducible(cuda):
    say("case determinism")
    v, f = mesh_case("sphere3")
    rng = np.random.default_rng(16)
    nv, nf, C, K = v.shape[0], f.shape[0], 64, 16
    x = dev(rng.uniform(-1, 1, (nf, C)), cuda, torch.float32)
    filt = dev(rng.normal(0, 0.5, (K, C, 1)), cuda, torch.float32)
    coeff = dev(rng.normal(0, 0.5, (nf, K)), cuda, torch.float32)
    gout = dev(rng.normal(0, 1, (nv, C)), cuda, torch.float32)
    ft, nfc, vm = dev(f, cuda), dev(S.vertex_facet_count(f, np.arange(nv), nv), cuda), dev(np.arange(nv, dtype=np.int32), cuda)
    runs = []
    for _ in range(3):
        o = mesh_conv3d.facet2vertex_forward(x, filt, coeff, ft, nfc, vm)
        gi, gf = mesh_conv3d.facet2vertex_backward(gout, x, filt, coeff, ft, nfc, vm)
        runs.append((o.clone(), gi.clone(), gf.clone()))
    torch.cuda.synchronize()
    for a, b in zip(runs[0], runs[1]):
        assert torch.equal(a, b)
    for a, b in zip(runs[0], runs[2]):
        assert torch.equal(a, b)


# ------------------------------------------------------------------ per-level inputs
@pytest.mark.parametrize("mesh", ["octa", "sphere3", "room_small"])
def test_adjface_count_and_triangle_geometry(cuda, mesh):
    from oracle import torch_ref as R
    from picassoplus_amd.mesh.pi_modules import geometry
    rng = np.random.default_rng(31)
    v, f = mesh_case(mesh)
    nv = v.shape[0]
    vt_map, nvo = strided_vt_map(rng, nv)
    got = geometry.count_vertex_adjface_(dev(f, cuda), dev(vt_map, cuda), torch.zeros(nvo, 3, device=cuda))
    ref = R.count_vertex_adjface(torch.from_numpy(f), torch.from_numpy(vt_map), nvo)
    assert torch.equal(got.cpu(), ref.to(torch.int32))
    assert int(got.sum()) == int((vt_map[f.reshape(-1)] >= 0).sum())
    # geometry: vertex rows carry extra columns (colour) after the position
    vx = np.concatenate([v, rng.uniform(0, 1, (nv, 3))], 1).astype(np.float32)
    geo = geometry.compute_triangle_geometry_(dev(vx, cuda), dev(f, cuda))
    torch.cuda.synchronize()
    p = vx[:, :3].astype(np.float64)
    raw = np.cross(p[f[:, 1]] - p[f[:, 0]], p[f[:, 2]] - p[f[:, 0]])
    ln = np.linalg.norm(raw, axis=1, keepdims=True)
    normal = raw / (ln + 1e-10)
    ref_geo = np.concatenate([normal, -(normal * p[f[:, 0]]).sum(1, keepdims=True), ln / 2], 1)
    # float32 cross products of thin or collapsed triangles cancel: direction and offset are compared
    # on the well-shaped facets, the area (absolute scale) on all of them
    e1, e2 = p[f[:, 1]] - p[f[:, 0]], p[f[:, 2]] - p[f[:, 0]]
    ok = ln[:, 0] > 0.1 * np.linalg.norm(e1, axis=1) * np.linalg.norm(e2, axis=1)
    assert ok.mean() > 0.5
    okt = torch.from_numpy(ok).to(cuda)
    assert_close(geo[okt][:, :4], ref_geo[ok][:, :4], "triangle normal and offset")
    assert_close(geo[:, 4], ref_geo[:, 4], "triangle area")
    assert_close(geo[okt][:, :3], R.face_normals(torch.from_numpy(p), torch.from_numpy(f)).numpy()[ok],
                 "normals vs oracle")


@pytest.mark.parametrize("mesh,L", [("octa", 3), ("sphere3", 3), ("room_small", 5), ("torus", None)])
def test_facet_frame_parity(cuda, mesh, L):
    """Geometry, oriented normals and their basis coefficients from one kernel against the oracle's three steps."""
    say("case facet_frame", mesh, L)
    from picassoplus_amd.mesh.pi_modules import geometry
    from oracle import torch_ref as R
    v, f = mesh_case(mesh)
    rng = np.random.default_rng(14)
    v = v + rng.normal(0, 0.3, 3)                                  # viewpoint off-centre
    vx = np.concatenate([v, rng.uniform(0, 1, (v.shape[0], 3))], 1).astype(np.float32)     # position + colour
    geo, nrm, coeff = geometry.facet_frame_(dev(vx, cuda), dev(f, cuda), L)
    torch.cuda.synchronize()
    assert torch.equal(geo, geometry.compute_triangle_geometry_(dev(vx, cuda), dev(f, cuda)))
    p = torch.from_numpy(vx[:, :3].astype(np.float64))
    n_ref = R.face_normals(p, torch.from_numpy(f))
    o_ref = R.oriented_normals(n_ref, p, torch.from_numpy(f)).numpy()
    centre = vx[:, :3].astype(np.float64)[f.astype(np.int64)].mean(1)
    # compared on well-shaped facets (float32 cross products of thin or collapsed triangles cancel) whose sign is
    # not a rounding matter
    pp = p.numpy()
    e1, e2 = pp[f[:, 1]] - pp[f[:, 0]], pp[f[:, 2]] - pp[f[:, 0]]
    shaped = np.linalg.norm(np.cross(e1, e2), axis=1) > 0.1 * np.linalg.norm(e1, axis=1) * np.linalg.norm(e2, axis=1)
    sure = shaped & (np.abs((centre * n_ref.numpy()).sum(1)) > 1e-4)
    assert sure.mean() > 0.5
    assert_close(nrm[torch.from_numpy(sure).to(cuda)], o_ref[sure], "oriented normals")
    assert torch.equal(nrm.abs(), geo[:, :3].abs())
    if L is None:
        assert coeff is None
    else:
        assert torch.equal(coeff, sph_harm_values(nrm, L))
        assert_close(coeff[torch.from_numpy(sure).to(cuda)], loops.sph_harm(o_ref[sure], L), "coefficients")
