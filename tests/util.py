"""Helpers shared by the tests: seeded cases and the parity metric."""
import numpy as np
import torch

from picassoplus_amd import synthetic as S

TOL_F32 = 1e-5   # max |y - y*| / max |y*| against the float64 oracle


def rel_err(y, ref):
    y = np.asarray(y, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert y.shape == ref.shape, (y.shape, ref.shape)
    if ref.size == 0:
        return 0.0
    den = np.abs(ref).max()
    num = np.abs(y - ref).max()
    return float(num / den) if den > 0 else float(num)


MEASURED = []    # (label, measured error, bound) of every parity assertion of the session, reported by conftest.py


def assert_close(y, ref, what, tol=TOL_F32):
    e = rel_err(y.detach().cpu().numpy() if isinstance(y, torch.Tensor) else y, ref)
    MEASURED.append((what, e, tol))
    assert e <= tol, "%s: max rel err %.3e > %.1e" % (what, e, tol)
    return e


# Second parity criterion of the convolutions: the build's error must not exceed `factor` times the error the float32
# loop oracle makes when it sums in the reference's order (both measured against the float64 answer).  Below two units
# of the last place of the largest value the comparison would measure the rounding of the result itself, not of the
# sums, hence the floor.  factor = 2 for vertex2facet and facet2vertex.  facet2facet is held to 3: the reference adds
# 16-term inner sums (over d) into each output, a blocked summation, while any matrix-core kernel runs ONE
# accumulator through all Cin * 16 terms of a row; that order alone costs the float32 matrix instruction 3 to 3.5
# times the reference order's error (the `generic` path, exact fp32 products), and the two-piece fp16
# kernels measure 1.1 to 2.6.
F32_FLOOR = 2.0 ** -22


def assert_as_good_as_f32(y, ref64, ref32, what, factor=2.0):
    """``y`` (GPU result) against the float64 oracle ``ref64``, relative to how far the float32 oracle ``ref32``
    (reference summation order) is from it: err(y) <= max(factor err(ref32), 2^-22).  Returns (err(y), err(ref32))."""
    e = rel_err(y.detach().cpu().numpy() if isinstance(y, torch.Tensor) else y, ref64)
    e32 = rel_err(ref32, ref64)
    # reported as the ratio to the float32 oracle's error (floored as the bound is) against the factor allowed
    MEASURED.append((what + (" [error / float32 oracle's error]" if factor else " [error / float32 oracle's error, cross-check path: reported only]"), e / max(e32, F32_FLOOR / (factor or 1.0)), factor or float("inf")))
    if factor is not None:
        assert e <= max(factor * e32, F32_FLOOR), "%s: error %.3e exceeds %g x the float32 oracle's %.3e" % (what, e, factor, e32)
    return e, e32


def dev(a, device, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(device)


def tiny_meshes():
    """Tetrahedron, octahedron and a 2x2 planar grid: (vertex, face) pairs."""
    tet_v = np.array([[1, 1, 1], [1, -1, -1], [-1, 1, -1], [-1, -1, 1]], np.float64)
    tet_f = np.array([[0, 1, 2], [0, 3, 1], [0, 2, 3], [1, 3, 2]], np.int32)
    oct_v = np.array([[1, 0, 0], [-1, 0, 0], [0, 1, 0], [0, -1, 0], [0, 0, 1], [0, 0, -1]], np.float64)
    oct_f = np.array([[0, 2, 4], [2, 1, 4], [1, 3, 4], [3, 0, 4], [2, 0, 5], [1, 2, 5], [3, 1, 5], [0, 3, 5]], np.int32)
    grid_v, grid_f = S.grid_patch(np.random.default_rng(0), 2, 2, (0, 0, 0), (1, 0, 0), (0, 1, 0))
    return {"tetra": (tet_v, tet_f), "octa": (oct_v, oct_f), "grid2": (grid_v, grid_f)}


def mesh_case(name, seed=0):
    """(vertex, face) for a named mesh."""
    tm = tiny_meshes()
    if name in tm:
        return tm[name]
    rng = np.random.default_rng(seed)
    if name.startswith("sphere"):
        return S.icosphere(int(name[6:]))
    if name == "torus":
        return S.torus(24, 16)
    if name == "room_small":
        return S.room(rng, scale=0.01)
    if name == "fans":
        # hubs of degree 20 and 11 (more than eight adjacency entries per vertex) next to low-degree rims
        def fan(n, base):
            hub = base
            rim = base + 1 + np.arange(n)
            return np.stack([np.full(n, hub), rim, np.roll(rim, -1)], 1)
        f = np.concatenate([fan(20, 0), fan(11, 21), fan(3, 33)]).astype(np.int32)
        v = rng.normal(0, 1, (37, 3))
        return v, f
    if name == "shapes_small":
        w = S.shapes_workload(seed=seed, n_meshes=2)
        return w["vertex"], w["face"]
    raise KeyError(name)


def strided_vt_map(rng, nv, keep=0.6):
    """Input->output vertex map with dropped vertices (-1), ascending on the kept ones."""
    kept = rng.random(nv) < keep
    kept[0] = True
    vt_map = np.where(kept, np.cumsum(kept) - 1, -1).astype(np.int32)
    return vt_map, int(kept.sum())


def texture_case(rng, nf, kmax=5, empty_frac=0.1):
    counts = rng.integers(1, kmax + 1, nf).astype(np.int32)
    counts[rng.random(nf) < empty_frac] = 0
    counts, bary, owner = S.texture_points(rng, nf, counts)
    return counts, bary, owner


TOL_BF16 = 1e-3   # reduced-precision variant: features in bf16 in HBM, fp32 accumulation


def to_bf16(a):
    """numpy float array -> the same values rounded to bf16 (nearest even), as float64."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).to(torch.float64).numpy()


def assert_close_bf16_store(y, ref, what, tol=TOL_BF16):
    """A result that left the kernel as bf16: within ``tol`` of the largest reference value before the final rounding
    to bf16, i.e. |y - ref| <= tol max|ref| + 2^-8 |ref| element by element.  bf16 keeps eight significant bits (one
    implicit, seven stored), so neighbouring values are 2^-7 of the binade's start apart: rounding to nearest moves a
    value by at most 2^-8 of its magnitude, a store that truncates by up to 2^-7 (test_host.py checks that such a
    store fails this criterion)."""
    y = y.detach().to(torch.float64).cpu().numpy() if isinstance(y, torch.Tensor) else np.asarray(y, np.float64)
    ref = np.asarray(ref, np.float64)
    assert y.shape == ref.shape, (y.shape, ref.shape)
    if ref.size == 0:
        return 0.0
    den = np.abs(ref).max()
    slack = np.abs(y - ref) - 2.0 ** -8 * np.abs(ref)
    e = float(slack.max() / den) if den > 0 else float(np.abs(y).max())
    MEASURED.append((what + " [bf16 store]", e, tol))
    assert e <= tol, "%s: error beyond the bf16 store rounding %.3e > %.1e of max|ref|" % (what, e, tol)
    return e
