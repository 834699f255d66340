"""ctypes binding of libpicasso_mesh.so (declared in include/picasso_mesh.h).

The library is the only compute path of this package: when it is missing the ops raise,
they never fall back to another implementation.
"""
import ctypes
import os

from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
# PICASSO_MESH_LIB points at an alternative build of the same ABI (kernel experiments)
LIB_PATH = os.environ.get("PICASSO_MESH_LIB") or os.path.join(_HERE, "csrc", "libpicasso_mesh.so")
ABI_VERSION = 21

P, I, L, Z = c_void_p, c_int, c_int64, c_size_t

# name -> (restype, argtypes); mirrors include/picasso_mesh.h one to one
SIGNATURES = {
    "pmesh_abi_version": (I, []),
    "pmesh_last_error": (c_char_p, []),
    "pmesh_vertex_csr_workspace_bytes": (Z, [L, L]),
    "pmesh_build_vertex_csr": (I, [P, P, L, L, L, P, P, P, Z, P]),
    "pmesh_cluster_csr_workspace_bytes": (Z, [L, L]),
    "pmesh_build_cluster_csr": (I, [P, P, L, L, P, P, P, Z, P]),
    "pmesh_v2f_fwd": (I, [P, P, P, P, L, L, I, I, P]),
    "pmesh_v2f_bwd_workspace_bytes": (Z, [I, I]),
    "pmesh_v2f_bwd": (I, [P, P, P, P, P, P, P, P, P, Z, L, L, I, I, P]),
    "pmesh_f2v_fwd": (I, [P, P, P, P, P, P, P, L, L, I, I, I, P]),
    "pmesh_f2v_bwd_workspace_bytes": (Z, [I, I, I]),
    "pmesh_f2v_bwd": (I, [P, P, P, P, P, P, P, P, P, P, Z, L, L, L, I, I, I, P]),
    "pmesh_f2v_bwd_static_max_bytes": (Z, []),
    "pmesh_f2v_bwd_static": (I, [P, P, P, P, P, P, P, P, P, L, L, L, I, I, I, P]),
    "pmesh_f2f_fwd_workspace_bytes": (Z, [I, I, I]),
    "pmesh_index_csr_workspace_bytes": (Z, [L, L]),
    "pmesh_build_index_csr": (I, [P, I, L, L, P, P, P, Z, P]),
    "pmesh_point_range_count": (I, [P, P, P, P, I, L, L, ctypes.c_float, I, P, P]),
    "pmesh_point_range_fill": (I, [P, P, P, P, I, L, L, ctypes.c_float, P, L, P, P, P]),
    "pmesh_point_cube_count": (I, [P, P, P, P, I, L, L, ctypes.c_float, I, P, P]),
    "pmesh_point_cube_fill": (I, [P, P, P, P, I, L, L, ctypes.c_float, I, P, L, P, P]),
    "pmesh_point_grid_workspace_bytes": (Z, [L]),
    "pmesh_point_grid_build": (I, [P, P, I, L, ctypes.c_float, P, Z, P]),
    "pmesh_point_range_count_grid": (I, [P, P, P, P, P, I, L, L, ctypes.c_float, I, P, P]),
    "pmesh_point_range_fill_grid": (I, [P, P, P, P, P, I, L, L, ctypes.c_float, P, L, P, P, P]),
    "pmesh_point_cube_count_grid": (I, [P, P, P, P, P, I, L, L, ctypes.c_float, I, P, P]),
    "pmesh_point_cube_fill_grid": (I, [P, P, P, P, P, I, L, L, ctypes.c_float, I, P, L, P, P]),
    "pmesh_point_knn3": (I, [P, P, P, P, I, L, L, P, P, P]),
    "pmesh_point_knn3_grid": (I, [P, P, P, P, P, I, L, L, P, P, P]),
    "pmesh_point_fps": (I, [P, P, P, I, L, L, P, P, P]),
    "pmesh_point_sph3d_kernel": (I, [P, P, P, P, L, L, L, I, I, I, ctypes.c_float, P, P]),
    "pmesh_point_fuzzy_sph3d_kernel": (I, [P, P, P, P, L, L, L, I, I, I, ctypes.c_float, P, P, P]),
    "pmesh_point_conv_fwd": (I, [P, P, P, P, P, P, P, P, P, L, L, L, I, I, I, I, P]),
    "pmesh_point_conv_bwd_workspace_bytes": (Z, [L, I, I, I]),
    "pmesh_point_conv_bwd": (I, [P, P, P, P, P, P, P, P, P, P, P, P, Z, L, L, L, I, I, I, I, P]),
    "pmesh_point_pool_max_fwd": (I, [P, P, P, P, P, P, L, L, L, I, P]),
    "pmesh_point_pool_max_bwd": (I, [P, P, P, P, P, P, L, L, L, I, P]),
    "pmesh_point_pool_avg_fwd": (I, [P, P, P, P, P, P, L, L, L, I, P]),
    "pmesh_point_pool_avg_bwd": (I, [P, P, P, P, P, P, L, L, L, I, P]),
    "pmesh_point_unpool_fwd": (I, [P, P, P, P, L, L, I, I, P]),
    "pmesh_point_unpool_bwd": (I, [P, P, P, P, P, L, L, I, I, P]),
    "pmesh_f2f_fwd": (I, [P, P, P, P, P, P, P, Z, L, L, I, I, I, P]),
    "pmesh_f2f_fwd_act": (I, [P, P, P, P, P, P, P, P, I, P, P, P, Z, L, L, I, I, I, P]),
    "pmesh_facet_order_workspace_bytes": (Z, [L]),
    "pmesh_build_facet_order": (I, [P, L, L, P, P, Z, P]),
    "pmesh_f2f_bwd_workspace_bytes": (Z, [I, I, I]),
    "pmesh_f2f_bwd_workspace_bytes_for": (Z, [L, I, I, I]),
    "pmesh_reload_options": (None, []),
    "pmesh_f2f_bwd": (I, [P, P, P, P, P, P, P, P, P, Z, L, L, I, I, I, P]),
    "pmesh_f2f_bwd_texture": (I, [P, P, P, P, P, P, P, Z, L, L, I, I, I, P]),
    "pmesh_f2f_bwd_texture_onto": (I, [P, P, P, P, P, P, P, Z, L, L, I, I, I, P]),
    "pmesh_f2f_bwd_texture_onto_supported": (I, [P, P, P, I, I]),
    "pmesh_f2f_bwd_filter": (I, [P, P, P, P, P, P, P, Z, L, L, I, I, I, P]),
    "pmesh_f2f_bwd_bf16_workspace_bytes": (Z, [L, L, I, I, I]),
    "pmesh_f2f_fwd_bf16": (I, [P, P, P, P, P, P, P, Z, L, L, I, I, I, P]),
    "pmesh_f2f_bwd_texture_bf16": (I, [P, P, P, P, P, P, P, Z, L, L, I, I, I, P]),
    "pmesh_f2f_bwd_filter_bf16": (I, [P, P, P, P, P, P, P, Z, L, L, I, I, I, P]),
    "pmesh_f2v_fwd_bf16": (I, [P, P, P, P, P, P, P, L, L, I, I, I, P]),
    "pmesh_f2v_bwd_bf16": (I, [P, P, P, P, P, P, P, P, P, P, Z, L, L, L, I, I, I, P]),
    "pmesh_pool_max_fwd": (I, [P, P, P, P, P, L, L, I, P]),
    "pmesh_pool_max_bwd": (I, [P, P, P, P, P, L, L, I, P]),
    "pmesh_pool_avg_fwd": (I, [P, P, P, P, P, L, L, I, P]),
    "pmesh_pool_avg_bwd": (I, [P, P, P, P, L, L, I, P]),
    "pmesh_unpool_fwd": (I, [P, P, P, P, L, L, I, P]),
    "pmesh_unpool_bwd": (I, [P, P, P, P, L, L, I, P]),
    "pmesh_count_vertex_adjface": (I, [P, P, L, P]),
    "pmesh_triangle_geometry": (I, [P, P, P, L, L, I, P]),
    "pmesh_sph_harm": (I, [P, P, L, I, P]),
    "pmesh_facet_frame": (I, [P, P, P, P, P, L, L, I, I, P]),
    "pmesh_texture_fwd": (I, [P, P, P, P, P, P, L, L, L, I, I, P]),
    "pmesh_texture_bwd": (I, [P, P, P, P, P, P, L, L, L, I, P]),
    "pmesh_combine_clusters": (I, [P, P, P, P, P, P, P, L, L, P]),
    "pmesh_vertex_quadrics": (I, [P, P, P, P, L, I, P]),
    "pmesh_boundary_quadrics": (I, [P, P, P, P, P, P, L, I, I, c_float, P]),
    "pmesh_edge_costs": (I, [P, P, P, P, P, L, I, P]),
    "pmesh_cluster_vertices_host": (I, [P, P, L, I, I, I, P]),
    "pmesh_edge_list_count": (I, [P, P, P, L, L, P, P, P, P]),
    "pmesh_edge_list_fill": (I, [P, P, P, L, L, P, P, P, P, P, P, P, P]),
    "pmesh_simplify_faces": (I, [P, P, L, L, P, P, P, P, P]),
    "pmesh_simplify_renumber": (I, [P, P, P, P, L, L, P, P, P]),
    "pmesh_cluster_match": (I, [P, P, P, L, L, P, P, P, P, I, P]),
    "pmesh_contraction_keys": (I, [P, P, P, P, L, I, P, P]),
    "pmesh_cluster_ranks": (I, [P, P, L, P, P, P]),
    "pmesh_cluster_flags_by_rank": (I, [P, P, L, P, P]),
    "pmesh_cluster_cut": (I, [P, P, P, P, P, P, L, I, P, P, P, P]),
    "pmesh_cluster_contract_pairs": (I, [P, P, P, L, P, P]),
    "pmesh_cluster_attach_propose": (I, [P, P, P, P, P, L, L, P, P, P, P]),
    "pmesh_cluster_attach": (I, [P, P, P, P, L, P, P, P, P]),
    "pmesh_dense_fwd": (I, [P, P, P, P, P, I, P, P, L, I, I, P]),
    "pmesh_v2f_dense_fwd": (I, [P, P, P, P, P, P, P, I, P, P, P, L, L, I, I, P]),
    "pmesh_f2v_dense_supported": (I, [L, I, I, I, I, P]),
    "pmesh_f2v_dense_fwd_workspace_bytes": (Z, [I, I, I]),
    "pmesh_f2v_dense_fwd": (I, [P, P, P, P, P, P, P, P, P, P, I, P, P, P, P, Z, L, L, I, I, I, I, P]),
    "pmesh_dense_bwd_workspace_bytes": (Z, [L, I, I]),
    "pmesh_dense_bwd": (I, [P, P, P, P, P, P, P, P, P, Z, L, I, I, P]),
    "pmesh_bias_act_fwd": (I, [P, P, P, P, I, P, P, L, I, P]),
    "pmesh_bias_act_bwd_workspace_bytes": (Z, [I]),
    "pmesh_bias_act_bwd": (I, [P, P, P, P, P, P, Z, L, I, P]),
}

_lib = None


class NativeLibraryError(RuntimeError):
    pass


def load():
    """Load the shared library once; raise loudly when it is absent or stale."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise NativeLibraryError(
            "libpicasso_mesh.so is not built (%s). Build it with `python -m picassoplus_amd.build`; "
            "this package has no other compute path." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as exc:
            raise NativeLibraryError("libpicasso_mesh.so lacks symbol %s; rebuild it" % name) from exc
        fn.restype, fn.argtypes = res, args
    if lib.pmesh_abi_version() != ABI_VERSION:
        raise NativeLibraryError("libpicasso_mesh.so has ABI %d, binding expects %d; rebuild it"
                                 % (lib.pmesh_abi_version(), ABI_VERSION))
    _lib = lib
    return lib


_call_hook = None


def set_call_hook(hook):
    """Install ``hook(name, phase)`` (phase "begin"/"end") around every native call, or None.
    The benchmark uses it to bracket calls with HIP events on the launch stream."""
    global _call_hook
    _call_hook = hook


def call(name, *args):
    """Invoke an int-returning entry point; non-zero becomes RuntimeError(last error)."""
    lib = load()
    hook = _call_hook
    if hook is not None:
        hook(name, "begin")
    rc = getattr(lib, name)(*args)
    if hook is not None:
        hook(name, "end")
    if rc != 0:
        msg = lib.pmesh_last_error()
        raise RuntimeError("%s failed: %s" % (name, msg.decode() if msg else "unknown error"))


def call_many(name, arg_lists, workers=8):
    """Invoke a HOST-side int-returning entry point once per argument list, on a small thread pool (ctypes releases
    the interpreter lock during a foreign call; the library's error text is per thread and is read on the thread
    that failed).  The call hook sees one begin / end pair around all of them."""
    lib = load()
    fn = getattr(lib, name)
    hook = _call_hook
    if hook is not None:
        hook(name, "begin")

    def one(args):
        rc = fn(*args)
        if rc != 0:
            msg = lib.pmesh_last_error()
            return msg.decode() if msg else "unknown error"
        return None

    if len(arg_lists) <= 1 or workers <= 1:
        errors = [one(a) for a in arg_lists]
    else:
        from concurrent.futures import ThreadPoolExecutor
        with ThreadPoolExecutor(max_workers=min(workers, len(arg_lists))) as pool:
            errors = list(pool.map(one, arg_lists))
    if hook is not None:
        hook(name, "end")
    for e in errors:
        if e is not None:
            raise RuntimeError("%s failed: %s" % (name, e))


def reload_options():
    """Make the library read its PMESH_* switches from the environment again (it reads them once, at its first
    call): for tests and benchmarks that change them inside one process."""
    load().pmesh_reload_options()


def query(name, *args):
    """Invoke a size query (host only)."""
    return int(getattr(load(), name)(*args))
