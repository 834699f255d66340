"""Parity of the native pointwise tail (matmul + bias + ReLU [+ frozen batch norm] and its gradients) with the
float64 oracle (oracle/torch_ref.py: dense_tail_fwd / dense_tail_bwd), through the Python ops and the modules
that use it.  Bar: within 1e-5 of max |reference|."""
import sys

import numpy as np
import pytest
import torch
import torch.nn as nn

from oracle import torch_ref
from picassoplus_amd.mesh import layers
from picassoplus_amd.mesh.pi_modules import dense
from util import assert_close

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


SHAPES = [(1, 1, 1), (33, 3, 13), (64, 8, 32), (1000, 64, 64), (257, 96, 20), (70, 130, 257), (4099, 128, 128),
          (100, 896, 40), (300, 256, 256), (515, 36, 64), (2048, 32, 96), (129, 448, 128), (95, 6, 5)]


def _case(seed, n, ci, co):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n, ci, dtype=torch.float64, generator=g)
    w = torch.randn(ci, co, dtype=torch.float64, generator=g) / np.sqrt(ci)
    b = torch.randn(co, dtype=torch.float64, generator=g)
    go = torch.randn(n, co, dtype=torch.float64, generator=g)
    return x, w, b, go


@pytest.fixture(params=["split_bf16", "fp32_mfma"])
def product_path(request, native_options):
    """The row kernels multiply on the bf16 matrix instruction with operands split in three (default) or, behind
    PMESH_DENSE_FP32MFMA=1, on the fp32 matrix instruction."""
    native_options(PMESH_DENSE_FP32MFMA="1" if request.param == "fp32_mfma" else "0")
    return request.param


@pytest.mark.parametrize("n,ci,co", SHAPES)
@pytest.mark.parametrize("relu", [True, False])
def test_dense_tail_forward_backward(cuda, product_path, n, ci, co, relu):
    say("case dense_tail", product_path, n, ci, co, relu)
    x, w, b, go = _case(n + ci, n, ci, co)
    f = lambda t: t.to(cuda, torch.float32).contiguous()
    xd, wd, bd, god = f(x), f(w), f(b), f(go)
    # the oracle sees the float32-rounded operands, so the mask of the ReLU is the same one
    x, w, b, go = xd.double().cpu(), wd.double().cpu(), bd.double().cpu(), god.double().cpu()
    out = dense.dense_tail_forward(xd, wd, bd, relu)
    ref = torch_ref.dense_tail_fwd(x, w, b, relu)
    torch.cuda.synchronize()
    assert_close(out, ref.numpy(), "dense forward")
    # entries whose float64 pre-activation is within rounding of zero may land on either side of the ReLU
    z = x @ w + b
    safe = (z.abs() > 1e-5 * z.abs().max()) | (not relu)
    out64 = torch.where(safe, ref, out.double().cpu())
    gx, gw, gb = dense.dense_tail_backward(god, xd, wd, out if relu else None)
    rx, rw, rb = torch_ref.dense_tail_bwd(go, x, w, out64 if relu else None)
    torch.cuda.synchronize()
    assert_close(gx, rx.numpy(), "dense grad_input")
    assert_close(gw, rw.numpy(), "dense grad_weight")
    assert_close(gb, rb.numpy(), "dense grad_bias")
    gx2, gw2, gb2 = dense.dense_tail_backward(god, xd, wd, out if relu else None, need_input=False)
    torch.cuda.synchronize()
    assert gx2 is None and torch.equal(gw2, gw) and torch.equal(gb2, gb)
    if relu:
        # the bit form of the ReLU mask: same output, bits = (out > 0), and the very same gradients from it
        out_b, bits = dense.dense_tail_forward(xd, wd, bd, True, with_bits=True)
        assert torch.equal(out_b, out) and bits.shape == (n, (co + 31) // 32) and bits.dtype == torch.int32
        cols = torch.arange(co, device=cuda)
        unpacked = (bits[:, cols // 32] >> (cols % 32)) & 1
        assert torch.equal(unpacked.bool(), out > 0)
        if co % 32:
            assert int((bits[:, -1].long() & 0xFFFFFFFF).max()) < (1 << (co % 32))          # no stray bits past Co
        gx3, gw3, gb3 = dense.dense_tail_backward(god, xd, wd, None, relu_bits=bits)
        torch.cuda.synchronize()
        assert torch.equal(gx3, gx) and torch.equal(gw3, gw) and torch.equal(gb3, gb)


def test_dense_tail_frozen_norm_and_missing_operands(cuda):
    say("case dense_tail frozen norm")
    x, w, b, _ = _case(5, 777, 64, 48)
    g = torch.Generator().manual_seed(6)
    scale = torch.randn(48, dtype=torch.float64, generator=g)
    shift = torch.randn(48, dtype=torch.float64, generator=g)
    f = lambda t: t.to(cuda, torch.float32).contiguous()
    xd, wd, bd, sd, hd = f(x), f(w), f(b), f(scale), f(shift)
    x, w, b, scale, shift = (t.double().cpu() for t in (xd, wd, bd, sd, hd))
    assert_close(dense.dense_tail_forward(xd, wd, bd, True, sd, hd),
                 torch_ref.dense_tail_fwd(x, w, b, True, scale, shift).numpy(), "relu + scale/shift")
    assert_close(dense.dense_tail_forward(xd, wd, None, False, sd, None),
                 torch_ref.dense_tail_fwd(x, w, None, False, scale, None).numpy(), "scale only")
    assert_close(dense.dense_tail_forward(xd, wd, None, False),
                 (x @ w).numpy(), "plain product")


def test_dense_tail_unaligned_rows_and_empty(cuda):
    say("case dense_tail unaligned / empty")
    x, w, b, go = _case(9, 301, 64, 64)
    f = lambda t: t.to(cuda, torch.float32).contiguous()
    # a view one float past an aligned base: rows are 4-byte aligned only
    flat = torch.empty(301 * 64 + 1, dtype=torch.float32, device=cuda)
    xd = flat[1:].view(301, 64)
    xd.copy_(f(x))
    assert xd.data_ptr() % 16 == 4 and xd.is_contiguous()
    wd, bd, god = f(w), f(b), f(go)
    x, w, b, go = (t.double().cpu() for t in (xd, wd, bd, god))
    out = dense.dense_tail_forward(xd, wd, bd, False)
    assert_close(out, torch_ref.dense_tail_fwd(x, w, b, False).numpy(), "unaligned forward")
    gx, gw, gb = dense.dense_tail_backward(god, xd, wd, None)
    rx, rw, rb = torch_ref.dense_tail_bwd(go, x, w, None)
    assert_close(gx, rx.numpy(), "unaligned grad_input")
    assert_close(gw, rw.numpy(), "unaligned grad_weight")
    assert_close(gb, rb.numpy(), "unaligned grad_bias")
    e = torch.empty(0, 64, device=cuda)
    assert dense.dense_tail_forward(e, wd, bd, True).shape == (0, 64)
    gx, gw, gb = dense.dense_tail_backward(torch.empty(0, 64, device=cuda), e, wd, None)
    torch.cuda.synchronize()
    assert gx.shape == (0, 64) and float(gw.abs().max()) == 0.0 and float(gb.abs().max()) == 0.0
    with pytest.raises(RuntimeError):
        dense.dense_tail_forward(xd, wd[:32].contiguous(), bd, True)
    with pytest.raises(RuntimeError):
        dense.dense_tail_forward(torch.randn(4, 897, device=cuda), torch.randn(897, 8, device=cuda), None, True)


def test_dense_tail_is_deterministic(cuda):
    say("case dense_tail deterministic")
    x, w, b, go = _case(13, 20000, 64, 64)
    f = lambda t: t.to(cuda, torch.float32).contiguous()
    xd, wd, bd, god = f(x), f(w), f(b), f(go)
    out = dense.dense_tail_forward(xd, wd, bd, True)
    a = dense.dense_tail_backward(god, xd, wd, out)
    for _ in range(3):
        bgrads = dense.dense_tail_backward(god, xd, wd, out)
        assert all(torch.equal(p, q) for p, q in zip(a, bgrads))


@pytest.mark.parametrize("act", ["relu", "none", "tanh"])
@pytest.mark.parametrize("with_bn", [True, False])
def test_per_item_module_train_and_eval(cuda, act, with_bn):
    """PerItemConv3d (picasso/mesh/layers.py:198-239) against the same composition in float64: training mode
    with gradients, then evaluation mode without (frozen batch norm inside the native pass)."""
    say("case per_item module", act, with_bn)
    torch.manual_seed(17)
    fn = {"relu": nn.ReLU(), "none": None, "tanh": nn.Tanh()}[act]
    mod = layers.PerItemConv3d(24, 40, activation_fn=fn, with_bn=with_bn).to(cuda).train()
    with torch.no_grad():
        mod.biases.add_(0.1 * torch.randn_like(mod.biases))
    import copy
    mod64 = copy.deepcopy(mod).cpu().double().train()
    x = torch.randn(333, 24)
    g = torch.randn(333, 40)

    def ref(m, t):
        y = t @ m.weights + m.biases
        if m.activation_fn is not None:
            y = m.activation_fn(y)
        return m.BatchNorm(y) if m.with_bn else y

    xg = x.to(cuda).requires_grad_(True)
    out = mod(xg)
    out.backward(g.to(cuda))
    x64 = x.double().requires_grad_(True)
    y = ref(mod64, x64)
    y.backward(g.double())
    torch.cuda.synchronize()
    assert_close(out, y.detach().numpy(), "PerItemConv3d output")
    assert_close(xg.grad, x64.grad.numpy(), "PerItemConv3d grad_input")
    for (n, p), (_, q) in zip(mod.named_parameters(), mod64.named_parameters()):
        if n == "biases" and with_bn and fn is None:
            # a batch norm straight after the bias removes it: the exact gradient is zero
            assert float(p.grad.abs().max()) < 1e-3 and float(q.grad.abs().max()) < 1e-9
            continue
        assert_close(p.grad, q.grad.numpy(), "grad of " + n)
    mod.eval(); mod64.eval()
    with torch.no_grad():
        assert_close(mod(x.to(cuda)), ref(mod64, x.double()).numpy(), "PerItemConv3d eval output")
    # evaluation mode with gradients enabled keeps the batch norm outside the native pass and still agrees
    xg2 = x.to(cuda).requires_grad_(True)
    assert_close(mod(xg2), ref(mod64, x.double()).detach().numpy(), "PerItemConv3d eval output (grad mode)")


@pytest.mark.parametrize("n,c", [(1, 1), (77, 13), (1000, 64), (4099, 32), (300, 1024), (65, 4096), (50000, 96), (33, 6)])
@pytest.mark.parametrize("relu", [True, False])
def test_bias_act_forward_backward(cuda, n, c, relu):
    say("case bias_act", n, c, relu)
    g = torch.Generator().manual_seed(n + c)
    f = lambda t: t.to(cuda, torch.float32).contiguous()
    xd, bd, god = f(torch.randn(n, c, generator=g)), f(torch.randn(c, generator=g)), f(torch.randn(n, c, generator=g))
    sd, hd = f(torch.randn(c, generator=g)), f(torch.randn(c, generator=g))
    x, b, go, sc, sh = (t.double().cpu() for t in (xd, bd, god, sd, hd))
    out = dense.bias_act_forward(xd, bd, relu)
    ref = torch_ref.bias_act_fwd(x, b, relu)
    # float32 x + b rounds once; where the float64 sum is within that rounding of zero the ReLU may differ
    assert_close(out, ref.numpy(), "bias_act forward")
    assert_close(dense.bias_act_forward(xd, bd, relu, sd, hd), torch_ref.bias_act_fwd(x, b, relu, sc, sh).numpy(),
                 "bias_act forward with scale/shift")
    gx, gb = dense.bias_act_backward(god, out if relu else None)
    rx, rb = torch_ref.bias_act_bwd(go, out.double().cpu() if relu else None)
    torch.cuda.synchronize()
    assert torch.equal(gx.cpu().double(), rx)                # a selection: exact
    assert_close(gb, rb.numpy(), "bias_act grad_bias")
    gx2, gb2 = dense.bias_act_backward(god, out if relu else None, need_input=False)
    assert gx2 is None and torch.equal(gb2, gb)
    if relu and c % 32 == 0:
        out_b, bits = dense.bias_act_forward(xd, bd, True, with_bits=True)
        cols = torch.arange(c, device=cuda)
        assert torch.equal(out_b, out) and torch.equal(((bits[:, cols // 32] >> (cols % 32)) & 1).bool(), out > 0)
        gx3, gb3 = dense.bias_act_backward(god, None, relu_bits=bits)
        torch.cuda.synchronize()
        assert torch.equal(gx3, gx) and torch.equal(gb3, gb)
    elif relu:
        with pytest.raises(RuntimeError):
            dense.bias_act_forward(xd, bd, True, with_bits=True)


@pytest.mark.parametrize("act", ["relu", "none", "tanh"])
def test_f2f_module_tail_eval_matches_float64(cuda, act):
    """F2FConv3d in evaluation mode without gradients folds its batch norm into the native bias pass; the same
    module in float64 on the CPU oracle ops is the answer."""
    import copy
    from util import texture_case
    say("case f2f module eval tail", act)
    torch.manual_seed(23)
    fn = {"relu": nn.ReLU(), "none": None, "tanh": nn.Tanh()}[act]
    rng = np.random.default_rng(23)
    counts, bary, _ = texture_case(rng, 300, kmax=6)
    mod = layers.F2FConv3d(8, 16, 3, activation_fn=fn).to(cuda)
    with torch.no_grad():
        mod.biases.add_(0.1 * torch.randn_like(mod.biases))
        mod.BatchNorm.running_mean.add_(0.05 * torch.randn_like(mod.BatchNorm.running_mean))
        mod.BatchNorm.running_var.mul_(1.5)
    mod.eval()
    mod64 = copy.deepcopy(mod).cpu().double().eval()
    tex = torch.from_numpy(rng.normal(0, 1, (int(counts.sum()), 8)))
    sh64 = torch_ref.sph_harm(torch.from_numpy(bary), 3)
    cum = torch.cumsum(torch.from_numpy(counts), 0, dtype=torch.int32)
    y = torch_ref.f2f_fwd(tex, mod64.weights, sh64, cum) + mod64.biases
    if fn is not None:
        y = fn(y)
    y = mod64.BatchNorm(y)
    with torch.no_grad():
        sh = layers.SphHarmCoeff(3)(torch.from_numpy(bary).to(cuda, torch.float32))
        out = mod(tex.to(cuda, torch.float32), sh, torch.from_numpy(counts).to(cuda))
    assert_close(out, y.detach().numpy(), "F2FConv3d eval output")


V2F_SHAPES = [("tetra", 4, 1), ("octa", 8, 32), ("sphere2", 32, 64), ("sphere3", 64, 64), ("torus", 64, 128), ("room_small", 96, 20),
              ("sphere2", 128, 300), ("fans", 12, 7), ("shapes_small", 256, 256)]


@pytest.mark.parametrize("mesh,c,co", V2F_SHAPES)
@pytest.mark.parametrize("relu", [True, False])
def test_v2f_dense_one_pass(cuda, product_path, mesh, c, co, relu):
    """vertex2facet + pointwise product + bias + ReLU as one kernel against the float64 oracle composition
    (oracle: v2f_fwd, then dense_tail_fwd), forward with and without the kept rows / mask bits / frozen norm, and all
    four gradients through autograd against the oracle's explicit backward formulas."""
    from oracle import loops
    from util import dev, mesh_case
    say("case v2f_dense", product_path, mesh, c, co, relu)
    v, f = mesh_case(mesh)
    nv, nf = v.shape[0], f.shape[0]
    rng = np.random.default_rng(c * 1000 + co)
    x = rng.uniform(-1, 1, (nv, c)).astype(np.float32)
    filt = rng.normal(0, 0.6, (3, c, 1)).astype(np.float32)
    w = (rng.normal(0, 1, (c, co)) / np.sqrt(c)).astype(np.float32)
    b = rng.normal(0, 0.3, co).astype(np.float32)
    g = rng.normal(0, 1, (nf, co)).astype(np.float32)
    xd, fd, wd, bd, gd, face = (dev(a, cuda) for a in (x, filt, w, b, g, f))
    rows64 = loops.v2f_fwd(x.astype(np.float64), filt.astype(np.float64), f)
    T = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.float64))
    ref = torch_ref.dense_tail_fwd(T(rows64), T(w), T(b), relu).numpy()
    out = dense.v2f_dense_forward(xd, fd, face, wd, bd, relu)
    out2, bits, rows = dense.v2f_dense_forward(xd, fd, face, wd, bd, relu, with_bits=True, keep_rows=True)
    torch.cuda.synchronize()
    assert_close(out, ref, "v2f_dense forward")
    assert torch.equal(out, out2)
    assert_close(rows, rows64, "v2f_dense kept rows")
    cols = torch.arange(co, device=cuda)
    if relu:
        assert torch.equal(((bits[:, cols // 32] >> (cols % 32)) & 1).bool(), out > 0)
    # the same bits as the two native passes it replaces make
    from picassoplus_amd.mesh.pi_modules import mesh_conv3d
    two = dense.dense_tail_forward(mesh_conv3d.vertex2facet_forward(xd, fd, face), wd, bd, relu)
    assert_close(out, two.double().cpu().numpy(), "v2f_dense against the two passes", 2e-6)
    scale, shift = dev(rng.uniform(0.5, 2, co).astype(np.float32), cuda), dev(rng.normal(0, 1, co).astype(np.float32), cuda)
    outn = dense.v2f_dense_forward(xd, fd, face, wd, bd, relu, scale, shift)
    assert_close(outn, ref * scale.double().cpu().numpy() + shift.double().cpu().numpy(), "v2f_dense with scale/shift")
    # gradients
    xg, fg, wg, bg = (t.clone().requires_grad_(True) for t in (xd, fd, wd, bd))
    y = dense.v2f_dense(xg, fg, face, wg, bg, relu)
    assert torch.equal(y.detach(), out)
    y.backward(gd)
    torch.cuda.synchronize()
    z = rows64 @ w.astype(np.float64) + b
    safe = (np.abs(z) > 1e-5 * np.abs(z).max()) | (not relu)
    out64 = np.where(safe, ref, out.double().cpu().numpy())
    grows, gw, gb = torch_ref.dense_tail_bwd(T(g), T(rows64), T(w), T(out64) if relu else None)
    gx, gf = loops.v2f_bwd(grows.numpy(), x.astype(np.float64), filt.astype(np.float64), f)
    assert_close(xg.grad, gx, "v2f_dense grad_input")
    assert_close(fg.grad, gf, "v2f_dense grad_filter")
    assert_close(wg.grad, gw.numpy(), "v2f_dense grad_weight")
    assert_close(bg.grad, gb.numpy(), "v2f_dense grad_bias")
    # nothing is kept when no gradient is recorded
    with torch.no_grad():
        assert torch.equal(dense.v2f_dense(xd, fd, face, wd, bd, relu), out)


def test_v2f_module_takes_the_one_pass_form(cuda):
    """V2FConv3d calls one native forward where the reference runs the convolution and three PyTorch ops; other depth
    multipliers and activations keep the separate passes.  Both give the oracle's result (test_gpu_modules.py)."""
    from picassoplus_amd import _lib
    from util import dev, mesh_case
    v, f = mesh_case("sphere2")
    x = torch.randn(v.shape[0], 32, device=cuda)
    face = dev(f, cuda)
    calls = []
    _lib.set_call_hook(lambda name, phase: calls.append(name) if phase == "begin" else None)
    try:
        layers.V2FConv3d(32, 64, 3, with_bn=False).to(cuda)(x, face)
        one = list(calls)
        del calls[:]
        layers.V2FConv3d(32, 64, 3, depth_multiplier=2, with_bn=False).to(cuda)(x, face)
        two = list(calls)
    finally:
        _lib.set_call_hook(None)
    assert [c for c in one if c != "pmesh_sph_harm"] == ["pmesh_v2f_dense_fwd"], one      # (the corner basis, first call only)
    assert "pmesh_v2f_fwd" in two and "pmesh_dense_fwd" in two, two


def test_v2f_dense_empty_and_refused_shapes(cuda):
    """No facets: an empty result, nothing launched on bad memory; a channel count that is not a multiple of 4 and a face
    index outside the vertex range raise like the ops they replace."""
    x = torch.randn(10, 8, device=cuda)
    filt = torch.randn(3, 8, 1, device=cuda)
    w = torch.randn(8, 5, device=cuda)
    none = torch.zeros((0, 3), dtype=torch.int32, device=cuda)
    out, bits, rows = dense.v2f_dense_forward(x, filt, none, w, None, True, with_bits=True, keep_rows=True)
    assert out.shape == (0, 5) and bits.shape == (0, 1) and rows.shape == (0, 8)
    face = torch.tensor([[0, 1, 2], [3, 9, 4]], dtype=torch.int32, device=cuda)
    assert dense.v2f_dense_forward(x, filt, face, w).shape == (2, 5)
    with pytest.raises(RuntimeError):
        dense.v2f_dense_forward(x[:, :6].contiguous(), filt[:, :6].contiguous(), face, w[:6].contiguous())
    with pytest.raises(RuntimeError):
        dense.v2f_dense_forward(x, filt, torch.tensor([[0, 1, 10]], dtype=torch.int32, device=cuda), w)
    with pytest.raises(RuntimeError):
        dense.v2f_dense_forward(x.cpu(), filt, face, w)


F2V_DENSE_SHAPES = [("sphere2", 32, 1, 32, False), ("sphere3", 64, 1, 64, True), ("room_small", 64, 1, 64, False),
                    ("fans", 64, 1, 128, False), ("torus", 32, 2, 64, True), ("sphere3", 32, 1, 128, False),
                    ("tetra", 64, 1, 32, False), ("shapes_small", 16, 2, 32, True), ("octa", 64, 1, 64, True)]


@pytest.mark.parametrize("mesh,c,r,co,strided", F2V_DENSE_SHAPES)
@pytest.mark.parametrize("relu", [True, False])
def test_f2v_dense_one_pass(cuda, mesh, c, r, co, strided, relu):
    """facet2vertex + pointwise product + bias + ReLU as one kernel against the float64 oracle composition (oracle:
    f2v_fwd, then dense_tail_fwd): forward with and without the kept rows / mask bits / frozen norm, every gradient
    through autograd against the oracle's explicit backward formulas.  Vertex counts that are no multiple of 16 end
    on a partly filled tile; ``strided`` leaves output vertices without facets (their convolution rows are zero, their
    outputs the activated bias)."""
    from oracle import loops
    from picassoplus_amd import synthetic as S
    from util import dev, mesh_case, strided_vt_map
    say("case f2v_dense", mesh, c, r, co, strided, relu)
    v, f = mesh_case(mesh)
    nv, nf, K = v.shape[0], f.shape[0], 16
    rng = np.random.default_rng(c * 1000 + co + r)
    if strided:
        vt_map, nvo = strided_vt_map(rng, nv)
    else:
        vt_map, nvo = np.arange(nv, dtype=np.int32), nv
    nfc = np.maximum(S.vertex_facet_count(f, vt_map, nvo), 1)
    x = rng.uniform(-1, 1, (nf, c)).astype(np.float32)
    filt = rng.normal(0, 0.5, (K, c, r)).astype(np.float32)
    coeff = rng.normal(0, 0.5, (nf, K)).astype(np.float32)
    w = (rng.normal(0, 1, (c * r, co)) / np.sqrt(c * r)).astype(np.float32)
    b = rng.normal(0, 0.3, co).astype(np.float32)
    g = rng.normal(0, 1, (nvo, co)).astype(np.float32)
    xd, fd, cd, wd, bd, gd, face, nfd, vmd = (dev(a, cuda) for a in (x, filt, coeff, w, b, g, f, nfc, vt_map))
    f64 = np.float64
    rows64 = loops.f2v_fwd(x.astype(f64), filt.astype(f64), coeff.astype(f64), f, nfc, vt_map)
    T = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.float64))
    ref = torch_ref.dense_tail_fwd(T(rows64), T(w), T(b), relu).numpy()
    assert dense.f2v_dense_supported(xd, fd, cd, wd)
    out = dense.f2v_dense_forward(xd, fd, cd, face, nfd, vmd, wd, bd, relu)
    out2, bits, rows = dense.f2v_dense_forward(xd, fd, cd, face, nfd, vmd, wd, bd, relu, with_bits=True, keep_rows=True)
    torch.cuda.synchronize()
    assert_close(out, ref, "f2v_dense forward")
    assert torch.equal(out, out2)
    assert_close(rows, rows64, "f2v_dense kept rows")
    # the kept rows are the rows of the convolution kernel, bit for bit
    from picassoplus_amd.mesh.pi_modules import mesh_conv3d
    conv = mesh_conv3d.facet2vertex_forward(xd, fd, cd, face, nfd, vmd)
    assert torch.equal(rows, conv)
    cols = torch.arange(co, device=cuda)
    if relu:
        assert torch.equal(((bits[:, cols // 32] >> (cols % 32)) & 1).bool(), out > 0)
    f32 = np.float32
    rows32 = loops.f2v_fwd(x, filt, coeff, f, nfc, vt_map, dtype=f32)
    z32 = rows32 @ w + b
    from util import assert_as_good_as_f32
    assert_as_good_as_f32(out, ref, np.maximum(z32, 0) if relu else z32, "f2v_dense forward")
    scale, shift = dev(rng.uniform(0.5, 2, co).astype(np.float32), cuda), dev(rng.normal(0, 1, co).astype(np.float32), cuda)
    outn = dense.f2v_dense_forward(xd, fd, cd, face, nfd, vmd, wd, bd, relu, scale, shift)
    assert_close(outn, ref * scale.double().cpu().numpy() + shift.double().cpu().numpy(), "f2v_dense with scale/shift")
    nob = dense.f2v_dense_forward(xd, fd, cd, face, nfd, vmd, wd, None, relu)
    assert_close(nob, torch_ref.dense_tail_fwd(T(rows64), T(w), T(np.zeros(co)), relu).numpy(), "f2v_dense without a bias")
    # gradients
    xg, fg, wg, bg = (t.clone().requires_grad_(True) for t in (xd, fd, wd, bd))
    y = dense.f2v_dense(xg, fg, cd, face, nfd, vmd, wg, bg, relu)
    assert torch.equal(y.detach(), out)
    y.backward(gd)
    torch.cuda.synchronize()
    z = rows64 @ w.astype(np.float64) + b
    safe = (np.abs(z) > 1e-5 * np.abs(z).max()) | (not relu)
    out64 = np.where(safe, ref, out.double().cpu().numpy())
    grows, gw, gb = torch_ref.dense_tail_bwd(T(g), T(rows64), T(w), T(out64) if relu else None)
    gx, gf = loops.f2v_bwd(grows.numpy(), x.astype(f64), filt.astype(f64), coeff.astype(f64), f, nfc, vt_map)
    assert_close(xg.grad, gx, "f2v_dense grad_input")
    assert_close(fg.grad, gf, "f2v_dense grad_filter")
    assert_close(wg.grad, gw.numpy(), "f2v_dense grad_weight")
    assert_close(bg.grad, gb.numpy(), "f2v_dense grad_bias")
    with torch.no_grad():
        assert torch.equal(dense.f2v_dense(xd, fd, cd, face, nfd, vmd, wd, bd, relu), out)


def test_f2v_module_takes_the_one_pass_form(cuda, native_options):
    """Without gradients to record, F2VConv3d calls one native forward where the reference runs the convolution and
    three PyTorch ops; a training step, shapes the one-pass kernel does not take (other channel counts or degrees) and
    the vector-ALU switch keep the separate passes."""
    from picassoplus_amd import _lib
    from picassoplus_amd import synthetic as S
    from util import dev, mesh_case
    native_options(PMESH_F2V_VALU="0", PMESH_F2V_FP32MFMA="0")
    v, f = mesh_case("sphere2")
    nv, nf = v.shape[0], f.shape[0]
    vt_map = np.arange(nv, dtype=np.int32)
    nfc = np.maximum(S.vertex_facet_count(f, vt_map, nv), 1)
    face, nfd, vmd = dev(f, cuda), dev(nfc, cuda), dev(vt_map, cuda)
    x = torch.randn(nf, 64, device=cuda)
    coeff = torch.randn(nf, 16, device=cuda)
    calls = []
    _lib.set_call_hook(lambda name, phase: calls.append(name) if phase == "begin" else None)
    try:
        mod = layers.F2VConv3d(64, 64, 3, with_bn=True).to(cuda).eval()
        with torch.no_grad():
            y_one = mod(x, face, nfd, vmd, coeff)
        one = list(calls)
        del calls[:]
        y_train = mod(x, face, nfd, vmd, coeff)                 # parameters require gradients: the two passes
        train = list(calls)
        del calls[:]
        with torch.no_grad():
            layers.F2VConv3d(64, 48, 3, with_bn=False).to(cuda)(x, face, nfd, vmd, coeff)
        two = list(calls)
        del calls[:]
        native_options(PMESH_F2V_VALU="1")
        with torch.no_grad():
            layers.F2VConv3d(64, 64, 3, with_bn=False).to(cuda)(x, face, nfd, vmd, coeff)
        valu = list(calls)
    finally:
        _lib.set_call_hook(None)
    assert "pmesh_f2v_dense_fwd" in one and "pmesh_f2v_fwd" not in one and "pmesh_dense_fwd" not in one, one
    assert "pmesh_f2v_fwd" in train and "pmesh_dense_fwd" in train and "pmesh_f2v_dense_fwd" not in train, train
    assert "pmesh_f2v_fwd" in two and "pmesh_dense_fwd" in two, two
    assert "pmesh_f2v_fwd" in valu and "pmesh_dense_fwd" in valu, valu
    # both forms of the same module agree to the parity bar
    assert_close(y_one, y_train.detach().double().cpu().numpy(), "F2VConv3d one pass against two", 2e-6)


def test_f2v_dense_refused_shapes(cuda):
    """Shapes outside the one-pass kernel's range are refused by the op (the module does not send them there) and no
    output vertices give an empty result."""
    from util import dev
    f = np.array([[0, 1, 2], [0, 2, 3]], np.int32)
    face, nfd, vmd = dev(f, cuda), dev(np.array([2, 1, 2, 1], np.int32), cuda), dev(np.arange(4, dtype=np.int32), cuda)
    x, filt, coeff = torch.randn(2, 64, device=cuda), torch.randn(16, 64, 1, device=cuda), torch.randn(2, 16, device=cuda)
    assert dense.f2v_dense_forward(x, filt, coeff, face, nfd, vmd, torch.randn(64, 64, device=cuda)).shape == (4, 64)
    assert not dense.f2v_dense_supported(x, filt, coeff, torch.randn(64, 48, device=cuda))
    with pytest.raises(RuntimeError):
        dense.f2v_dense_forward(x, filt, coeff, face, nfd, vmd, torch.randn(64, 48, device=cuda))
    with pytest.raises(RuntimeError):
        dense.f2v_dense_forward(x[:, :24].contiguous(), filt[:, :24].contiguous(), coeff, face, nfd, vmd, torch.randn(24, 64, device=cuda))
    with pytest.raises(RuntimeError):
        dense.f2v_dense_forward(x, torch.randn(9, 64, 1, device=cuda), coeff[:, :9].contiguous(), face, nfd, vmd,
                                torch.randn(64, 64, device=cuda))
    none = torch.zeros((0,), dtype=torch.int32, device=cuda)
    nowhere = torch.full((4,), -1, dtype=torch.int32, device=cuda)
    out, bits, rows = dense.f2v_dense_forward(x, filt, coeff, face, none, nowhere, torch.randn(64, 64, device=cuda), None, True,
                                              with_bits=True, keep_rows=True)
    assert out.shape == (0, 64) and bits.shape == (0, 2) and rows.shape == (0, 64)
