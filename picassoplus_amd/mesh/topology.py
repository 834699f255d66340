"""Sorted adjacency (CSR) of index tensors, built on the GPU once and reused.

The reference passes raw index tensors (``face``, ``vt_map``, ``vt_replace``) to every op
and scatters with float atomics.  Here the scatter ops are segmented reductions, which need
the transposed adjacency.  A network reuses the same index tensors for every convolution of
a mesh level, forward and backward (picasso/networks/pi2_blocks.py:89-92 in the reference),
so the adjacency is cached per index tensor.

Cache discipline
  key      storage address, shape, in-place version counter and device of every index tensor
           involved (plus the integer arguments).  Inference tensors carry no version counter;
           they cannot be modified outside inference mode, and their key uses -1.
  lifetime an entry holds WEAK references to its index tensors and dies with the first of them:
           a training loop that feeds fresh ``face`` / ``vt_map`` tensors every batch
           (picasso/mesh/fit.py:34-45, dataset_scene.py:87-111) keeps the adjacency of the
           batches still alive and nothing else.  While a tensor lives its storage address
           cannot be handed to another allocation, so a live key never names other data.
  size     the device arrays of all entries together stay below ``MAX_BYTES`` (environment
           variable PICASSO_MESH_CACHE_BYTES, default 2 GiB); the least recently used go first.
  streams  an entry remembers the stream it was built on and an event recorded behind the build;
           a consumer on another stream waits for that event (nothing is waited for once the
           event has completed, and nothing during stream capture, whose warm-up has run the build).
"""
import contextlib
import os
import threading
import weakref
from collections import OrderedDict

import torch

from .. import _lib

_LOCK = threading.RLock()        # re-entrant: a finaliser may run while the owner thread holds it
_CACHE = OrderedDict()           # key -> _Entry
_BYTES = 0
MAX_BYTES = int(os.environ.get("PICASSO_MESH_CACHE_BYTES", str(2 << 30)))


class _Entry:
    __slots__ = ("value", "nbytes", "stream", "event", "finalizers")

    def __init__(self, value, nbytes, stream, event):
        self.value, self.nbytes, self.stream, self.event, self.finalizers = value, nbytes, stream, event, []


def clear_cache():
    global _BYTES
    with _LOCK:
        _BLOCKS.clear()
        for e in _CACHE.values():
            for fin in e.finalizers:
                fin.detach()
        _CACHE.clear()
        _BYTES = 0


def cache_bytes():
    """Device bytes held by the cached adjacency arrays."""
    return _BYTES


def cache_entries():
    return len(_CACHE)


def _version(t):
    return t._version if not t.is_inference() else -1


def _key(kind, *tensors_and_ints):
    parts = [kind]
    for t in tensors_and_ints:
        if isinstance(t, torch.Tensor):
            parts.append((t.data_ptr(), tuple(t.shape), _version(t), t.device.index))
        else:
            parts.append(t)
    return tuple(parts)


def _drop(key):
    global _BYTES
    with _LOCK:
        e = _CACHE.pop(key, None)
        if e is not None:
            _BYTES -= e.nbytes
            for fin in e.finalizers:
                fin.detach()


def _lookup(key):
    """Cached value or None.  A hit on another stream than the builder's waits for the build."""
    with _LOCK:
        e = _CACHE.get(key)
        if e is None:
            return None
        _CACHE.move_to_end(key)
        ev = e.event
    if ev is not None:
        if ev.query():
            e.event = None
        elif not torch.cuda.is_current_stream_capturing():
            cur = torch.cuda.current_stream()
            if cur.cuda_stream != e.stream:
                cur.wait_event(ev)
    return e.value


def _store(key, value, owners, arrays=()):
    """``owners``: the index tensors the entry is valid for (weakly referenced); ``arrays``: the device arrays
    built for it (counted against MAX_BYTES; they are part of ``value``)."""
    global _BYTES
    nbytes = sum(int(a.numel()) * a.element_size() for a in arrays)
    event = stream = None
    if arrays and arrays[0].is_cuda and not torch.cuda.is_current_stream_capturing():
        cur = torch.cuda.current_stream(arrays[0].device)
        event, stream = torch.cuda.Event(), cur.cuda_stream
        event.record(cur)
    e = _Entry(value, nbytes, stream, event)
    with _LOCK:
        _drop(key)
        for t in owners:
            if t is not None:
                fin = weakref.finalize(t, _drop, key)
                fin.atexit = False
                e.finalizers.append(fin)
        _CACHE[key] = e
        _BYTES += nbytes
        while _BYTES > MAX_BYTES and len(_CACHE) > 1:
            _drop(next(iter(_CACHE)))


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def _checks_enabled():
    return os.environ.get("PICASSO_MESH_SKIP_CHECKS", "0") != "1"


_TRUST = threading.local()


@contextlib.contextmanager
def trusted_indices():
    """Inside this block the index tensors handed to the library are its own kernels' outputs (the rounds of a
    decimation): their range checks -- one reduction and one synchronisation each -- are skipped."""
    _TRUST.depth = getattr(_TRUST, "depth", 0) + 1
    try:
        yield
    finally:
        _TRUST.depth -= 1


def _check_range(name, t, lo, hi):
    """One-off validation of an index tensor (one reduction and one synchronisation; only on a cache miss,
    and not at all with PICASSO_MESH_SKIP_CHECKS=1 or inside ``trusted_indices``)."""
    if t.numel() == 0 or not _checks_enabled() or getattr(_TRUST, "depth", 0):
        return
    mn, mx = (int(x) for x in torch.aminmax(t))
    if mn < lo or mx >= hi:
        raise RuntimeError("%s holds indices in [%d, %d], valid range is [%d, %d)" % (name, mn, mx, lo, hi))


def vertex_csr(face, vt_map, n_rows):
    """Row v -> ascending list of entries e = 3*facet + corner landing on v.

    ``vt_map`` None keys entries by ``face`` itself (rows = input vertices); otherwise by
    ``vt_map[face]`` with negative values dropped (rows = output vertices).
    Returns (rowptr int32 (n_rows+1), colidx int32 (3*Nf)).
    """
    key = _key("v", face, vt_map, int(n_rows))
    hit = _lookup(key)
    if hit is not None:
        return hit
    nf = face.shape[0]
    n_keys = vt_map.shape[0] if vt_map is not None else n_rows
    _check_range("face", face, 0, n_keys)
    with torch.cuda.device(face.device):
        rowptr = torch.empty(n_rows + 1, dtype=torch.int32, device=face.device)
        colidx = torch.empty(3 * nf, dtype=torch.int32, device=face.device)
        ws_bytes = _lib.query("pmesh_vertex_csr_workspace_bytes", nf, n_rows)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=face.device)
        _lib.call("pmesh_build_vertex_csr", face.data_ptr(), vt_map.data_ptr() if vt_map is not None else None,
                  nf, n_keys if vt_map is not None else 0, n_rows, rowptr.data_ptr(), colidx.data_ptr(),
                  ws.data_ptr(), ws_bytes, _stream(face))
    _store(key, (rowptr, colidx), (face, vt_map), (rowptr, colidx))
    return rowptr, colidx


def cluster_csr(vt_replace, vt_map, n_coarse):
    """Coarse row -> ascending list of fine vertices of that decimation cluster.

    Returns (rowptr int32 (n_coarse+1), members int32 (n_fine)).
    """
    key = _key("c", vt_replace, vt_map, int(n_coarse))
    hit = _lookup(key)
    if hit is not None:
        return hit
    n_fine = vt_replace.shape[0]
    if vt_map.shape[0] != n_fine:
        raise RuntimeError("vt_replace and vt_map must have the same length")
    _check_range("vt_replace", vt_replace, -(n_fine - 1), max(n_fine, 1))
    with torch.cuda.device(vt_replace.device):
        rowptr = torch.empty(n_coarse + 1, dtype=torch.int32, device=vt_replace.device)
        members = torch.empty(n_fine, dtype=torch.int32, device=vt_replace.device)
        ws_bytes = _lib.query("pmesh_cluster_csr_workspace_bytes", n_fine, n_coarse)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=vt_replace.device)
        _lib.call("pmesh_build_cluster_csr", vt_replace.data_ptr(), vt_map.data_ptr(), n_fine, n_coarse,
                  rowptr.data_ptr(), members.data_ptr(), ws.data_ptr(), ws_bytes, _stream(vt_replace))
    _store(key, (rowptr, members), (vt_replace, vt_map), (rowptr, members))
    return rowptr, members


def index_csr(index, column, n_rows):
    """Row r -> ascending list of the entries i with ``index[i, column] == r`` (the point-cloud ops' pairs sorted by
    query or by database point); ``column`` None takes the flattened tensor itself as the keys.
    Returns (rowptr int32 (n_rows + 1), order int32 (n_entries))."""
    key = _key("i", index, -1 if column is None else int(column), int(n_rows))
    hit = _lookup(key)
    if hit is not None:
        return hit
    if column is None:
        n, stride, offset = index.numel(), 1, 0
    else:
        n, stride, offset = index.shape[0], index.shape[1], int(column)
    with torch.cuda.device(index.device):
        rowptr = torch.empty(n_rows + 1, dtype=torch.int32, device=index.device)
        order = torch.empty(n, dtype=torch.int32, device=index.device)
        ws_bytes = _lib.query("pmesh_index_csr_workspace_bytes", n, n_rows)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=index.device)
        _lib.call("pmesh_build_index_csr", index.data_ptr() + 4 * offset if n else None, stride, n, n_rows, rowptr.data_ptr(),
                  order.data_ptr(), ws.data_ptr(), ws_bytes, _stream(index))
    _store(key, (rowptr, order), (index,), (rowptr, order))
    return rowptr, order


def facet_order(cum_texture, n_points):
    """Permutation of the facets by their number of texture points (stable), from the running
    total ``cum_texture``; lets the facet2facet kernels give every wavefront facets of equal length."""
    key = _key("o", cum_texture, int(n_points))
    hit = _lookup(key)
    if hit is not None:
        return hit
    nf = cum_texture.shape[0]
    with torch.cuda.device(cum_texture.device):
        order = torch.empty(nf, dtype=torch.int32, device=cum_texture.device)
        ws_bytes = _lib.query("pmesh_facet_order_workspace_bytes", nf)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=cum_texture.device)
        _lib.call("pmesh_build_facet_order", cum_texture.data_ptr(), nf, int(n_points), order.data_ptr(),
                  ws.data_ptr(), ws_bytes, _stream(cum_texture))
    _store(key, order, (cum_texture,), (order,))
    return order


def running_total(num_texture):
    """Inclusive running total (int32) of the per-facet texture-point counts, the form facet2facet takes
    (picasso/mesh/layers.py:57 computes it in every forward); cached per counts tensor, so that the facet order
    built from it is found again too."""
    key = _key("t", num_texture)
    hit = _lookup(key)
    if hit is not None:
        return hit
    total = torch.cumsum(num_texture, dim=0, dtype=torch.int)
    _store(key, total, (num_texture,), (total,))
    return total


_BLOCKS = {}            # device index -> (key, [blocks]): the coefficient blocks of the tensor seen last on that device


def coefficient_blocks(coeff):
    """A (rows, K) coefficient tensor cut into ceil(K / 16) contiguous blocks of 16 columns, the last one padded
    with zeros: what the 16-coefficient matrix-core kernels take for other spherical-harmonic degrees.  The
    blocks of the tensor seen last on a device are kept (the forward and the backward pass of a layer, and the
    layers of one mesh level, hand in the same tensor), so that they are cut once and not once per native call;
    they go when the tensor does, or when another one takes their place."""
    key = _key("b", coeff)
    dev = coeff.device.index
    stream = torch.cuda.current_stream(coeff.device).cuda_stream if coeff.is_cuda else None
    with _LOCK:
        hit = _BLOCKS.get(dev)
        if hit is not None and hit[0] == key and hit[2] == stream:      # (another stream cuts its own: no event to wait for)
            return hit[1]
    K = coeff.shape[1]
    pad = torch.nn.functional.pad
    blocks = [coeff[:, 16 * j:16 * j + 16].contiguous() if 16 * j + 16 <= K else pad(coeff[:, 16 * j:], (0, 16 * j + 16 - K))
              for j in range((K + 15) // 16)]
    if torch.cuda.is_current_stream_capturing():
        return blocks                                   # (a capture keeps its own tensors alive; nothing to share)

    def forget(dev=dev, key=key):
        with _LOCK:
            if dev in _BLOCKS and _BLOCKS[dev][0] == key:
                del _BLOCKS[dev]

    with _LOCK:
        _BLOCKS[dev] = (key, blocks, stream)
    fin = weakref.finalize(coeff, forget)
    fin.atexit = False
    return blocks


def checked_once(kind, owners, extra, check):
    """Run ``check()`` unless the same tensors (and ``extra`` integers) passed it before."""
    key = _key(kind, *owners, *extra)
    if _lookup(key) is None:
        check()
        _store(key, True, owners)


def _check_range_cached(face, n_vertices):
    """Validate a facet tensor against a vertex count once per tensor."""
    checked_once("rf", (face,), (int(n_vertices),), lambda: _check_range("face", face, 0, n_vertices))


def _check_cluster_cached(vt_replace, vt_map):
    n_fine = vt_replace.shape[0]
    checked_once("rk", (vt_replace, vt_map), (),
                 lambda: _check_range("vt_replace", vt_replace, -(n_fine - 1), max(n_fine, 1)))
