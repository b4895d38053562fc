"""Loader and ctypes signatures of librocshmem_mi355x.so (see include/rocshmem_mi355x.h)."""
import ctypes as C
import os

from .build import LIB_PATH, build

vp, sz, i32, u32, u64, i64 = C.c_void_p, C.c_size_t, C.c_int, C.c_uint32, C.c_uint64, C.c_int64


class Launch(C.Structure):
    _fields_ = [("wgs_per_pe", i32), ("wg_size", i32), ("tile", sz), ("stream", vp)]


LP = C.POINTER(Launch)

# name -> (restype, argtypes); every symbol declared in include/rocshmem_mi355x.h
SIGNATURES = {
    "rsm_init": (i32, [i32, sz, i32, C.c_uint]),
    "rsm_finalize": (i32, []),
    "rsm_is_initialized": (i32, []),
    "rsm_last_error": (C.c_char_p, []),
    "rsm_n_pes": (i32, []),
    "rsm_num_blocks": (i32, []),
    "rsm_heap_size": (sz, []),
    "rsm_slice_stride": (sz, []),
    "rsm_malloc": (vp, [sz]),
    "rsm_free": (i32, [vp]),
    "rsm_heap_bytes_in_use": (sz, []),
    "rsm_ptr": (vp, [vp, i32]),
    "rsm_heap_base": (vp, [i32]),
    "rsm_state_units": (i32, []),
    "rsm_take_status": (i32, []),
    "rsm_set_pacing": (i32, [C.c_uint, C.c_uint]),
    "rsm_get_pacing": (i32, [C.POINTER(C.c_uint), C.POINTER(C.c_uint)]),
    "rsm_tune_reduce_pacing": (i32, [i32, i32, vp, vp, sz, i32, i32, i32, vp, LP, C.POINTER(C.c_uint),
                                     C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "rsm_team_world": (u64, []),
    "rsm_team_split_strided": (i32, [u64, i32, i32, i32, C.POINTER(u64)]),
    "rsm_team_destroy": (i32, [u64]),
    "rsm_team_n_pes": (i32, [u64]),
    "rsm_team_translate_pe": (i32, [u64, i32, u64]),
    "rsm_copy_to_device": (i32, [vp, vp, sz]),
    "rsm_copy_to_host": (i32, [vp, vp, sz]),
    "rsm_fill": (i32, [vp, i32, sz]),
    "rsm_synchronize": (i32, []),
    "rsm_stream_synchronize": (i32, [vp]),
    "rsm_device_alloc": (vp, [sz]),
    "rsm_device_free": (i32, [vp]),
    "rsm_stream_create": (vp, []),
    "rsm_stream_destroy": (i32, [vp]),
    "rsm_event_create": (vp, []),
    "rsm_event_destroy": (i32, [vp]),
    "rsm_event_record": (i32, [vp, vp]),
    "rsm_event_elapsed_ms": (i32, [vp, vp, C.POINTER(C.c_float)]),
    "rsm_capture_begin": (i32, [vp]),
    "rsm_capture_end": (vp, [vp]),
    "rsm_graph_launch": (i32, [vp, vp]),
    "rsm_graph_destroy": (i32, [vp]),
    "rsm_to_all": (i32, [i32, i32, vp, vp, sz, i32, i32, i32, vp, vp, LP]),
    "rsm_to_all_noalloc": (i32, [i32, i32, vp, vp, sz, i32, i32, i32, LP]),
    "rsm_to_all_team": (i32, [i32, i32, u64, vp, vp, sz, LP]),
    "rsm_rma": (i32, [i32, i32, vp, vp, sz, sz, sz, sz, i32, LP]),
    "rsm_stream_probe": (i32, [i32, vp, sz, vp, C.c_uint, LP]),
    "rsm_broadcast": (i32, [sz, vp, vp, sz, i32, i32, i32, i32, vp, LP]),
    "rsm_broadcast_team": (i32, [sz, u64, vp, vp, sz, i32, LP]),
    "rsm_alltoall": (i32, [sz, u64, vp, vp, sz, LP]),
    "rsm_fcollect": (i32, [sz, u64, vp, vp, sz, LP]),
    "rsm_barrier_all": (i32, [i32, LP]),
    "rsm_small_ops": (i32, [vp, sz, vp, LP]),
    "rsm_sq_flush_target": (i32, [i32, C.POINTER(C.c_uint64), C.POINTER(C.c_uint32)]),
    "rsm_sq_reset": (i32, []),
    "rsm_sq_read": (i32, [i32, i32, C.c_uint, vp]),
    "rsm_sq_image": (i32, [i32, i32, vp, sz]),
    "rsm_sq_state": (i32, [i32, i32, C.POINTER(u32), C.POINTER(u32), C.POINTER(u32), vp]),
    "rsm_sq_constants": (i32, [i32, i32, C.POINTER(u32), C.POINTER(u64), C.POINTER(u32),
                               C.POINTER(u32), C.POINTER(u64), C.POINTER(u32)]),
    "rsm_sq_rkey": (i32, [i32, C.POINTER(u32)]),
    "rsm_sq_consume": (i32, [i32, i32, vp, vp]),
    "rsm_sq_set_mode": (i32, [i32]),
    "rsm_sq_consumer_start": (i32, []),
    "rsm_sq_consumer_stop": (i32, [vp]),
    "rsm_sq_consumer_running": (i32, []),
    "rsm_cq_reader_state": (i32, [i32, i32, C.POINTER(u32), C.POINTER(u32), C.POINTER(u32)]),
    "rsm_sq_consumer_state": (i32, [i32, i32, C.POINTER(u32), C.POINTER(u32)]),
    "rsm_cq_image": (i32, [i32, i32, vp, sz]),
    "rsm_atomic_ret_image": (i32, [i32, i32, vp, sz]),
    "rsm_arena": (i32, [C.POINTER(vp), C.POINTER(sz), C.POINTER(sz)]),
    "rsm_kat_fetch_incr": (i32, [u64, i32, i32, vp, C.POINTER(u64)]),
    "rsm_kat_coalesce": (i32, [u64, vp, vp, vp, vp, vp, vp]),
    "rsm_host_alloc_create": (vp, [sz]),
    "rsm_host_alloc_destroy": (None, [vp]),
    "rsm_host_alloc_alloc": (sz, [vp, sz]),
    "rsm_host_alloc_free": (i32, [vp, sz]),
    "rsm_host_alloc_in_use": (sz, [vp]),
    "rsm_host_active_set_in_range": (i32, [i32, i32, i32, i32]),
}

_lib = None


def load():
    """Load the HIP library; there is no CPU fallback: a missing or unloadable
    library is an error."""
    global _lib
    if _lib is not None:
        return _lib
    # ROC_SHMEM_LIBRARY names a variant build of the same sources (csrc/Makefile: EXTRA=, LIB=)
    path = os.environ.get("ROC_SHMEM_LIBRARY") or LIB_PATH
    if path == LIB_PATH and not os.path.exists(LIB_PATH):
        build()
    lib = C.CDLL(path)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib
