"""ctypes binding of libbikv_pagecopy.so (declarations: include/bikv_pagecopy.h).

The library is the product; there is no Python or CPU fallback. Loading fails loudly when the shared
object has not been built, and every entry point raises RuntimeError with the library's own message
when it returns a negative code — the exception type the reference's pybind module raises from
std::runtime_error / TORCH_CHECK (Bi-KV/SharedMemory/CUDA_Shared/ipc_service.cpp:30-108,
copy_kernel.cu:78-79).
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libbikv_pagecopy.so")

MAX_DIM = 5
ABI_VERSION = 4

OK, EINVAL, EHIP, ESYS, ESTATE, EBOUNDS, ERANGE = 0, -1, -2, -3, -4, -5, -6
ST_SRC_RANGE, ST_DST_RANGE, ST_PAGE_ID = 1, 2, 4
LAYOUT_LAYER_MAJOR, LAYOUT_PAGE_MAJOR = 0, 1
HINT_NONE, HINT_LAYER_MAJOR, HINT_PAGE_MAJOR = 0, 1, 2
STAGE_PIPELINED, STAGE_DIRECT, STAGE_AUTO, STAGE_PIPELINED_KERNEL = 0, 1, 2, 3
TRACE_KINDS = ("kernel", "copy_d2h", "copy_h2d", "copy_kernel")
PLACE_SPREAD, PLACE_SEQUENTIAL = 0, 1


class PoolDesc(C.Structure):
    _fields_ = [
        ("device", C.c_int32),
        ("n_planes", C.c_int32),
        ("n_pages", C.c_int64),
        ("tile_bytes", C.c_int64),
        ("page_stride_bytes", C.c_int64),
        ("plane_base", C.POINTER(C.c_void_p)),
        ("scale_tile_bytes", C.c_int64),
        ("scale_page_stride_bytes", C.c_int64),
        ("scale_plane_base", C.POINTER(C.c_void_p)),
        ("row_bytes", C.c_int64),
        ("row_stride_bytes", C.c_int64),
    ]


class PageBatchDesc(C.Structure):
    _fields_ = [
        ("page_ids", C.c_void_p),
        ("slots", C.c_void_p),
        ("slot_strides", C.c_void_p),
        ("n_pages", C.c_int64),
        ("plane_begin", C.c_int32),
        ("plane_count", C.c_int32),
        ("slot_bias", C.c_int64),
        ("layout_hint", C.c_int32),
        ("reserved", C.c_int32),
    ]


class NHDDesc(C.Structure):
    _fields_ = [
        ("device", C.c_int32),
        ("n_layers", C.c_int32),
        ("kv_heads", C.c_int32),
        ("head_dim", C.c_int32),
        ("block_tokens", C.c_int32),
        ("elem_bytes", C.c_int32),
        ("n_blocks", C.c_int64),
        ("block_stride_elems", C.c_int64),
        ("kv_stride_elems", C.c_int64),
        ("token_stride_elems", C.c_int64),
        ("layer_base", C.POINTER(C.c_void_p)),
    ]


class AllocInfo(C.Structure):
    _fields_ = [("bytes", C.c_int64), ("chunk_bytes", C.c_int64), ("n_chunks", C.c_int32),
                ("n_other_half", C.c_int32), ("n_fillers", C.c_int32), ("n_reprobed", C.c_int32),
                ("seconds", C.c_double), ("pair_ms_same", C.c_float), ("pair_ms_other", C.c_float)]


class StageStats(C.Structure):
    _fields_ = [("bytes", C.c_int64), ("n_chunks", C.c_int64), ("wall_seconds", C.c_double)]


class TraceStep(C.Structure):
    _fields_ = [("lane", C.c_int32), ("kind", C.c_int32), ("bytes", C.c_int64), ("start_ms", C.c_float),
                ("end_ms", C.c_float)]


class TensorDimsC(C.Structure):
    _fields_ = [
        ("total_tokens", C.c_int64),
        ("head_size", C.c_int64),
        ("num_kv_heads", C.c_int64),
        ("num_layers", C.c_int64),
        ("kv_pair", C.c_int64),
    ]


class SharedControl(C.Structure):
    """Byte-for-byte the reference's SharedControl (ipc_wrapper.h:14-28); sizeof == 480."""

    _fields_ = [
        ("sem_start", C.c_ubyte * 32),
        ("sem_complete", C.c_ubyte * 32),
        ("dtype_code", C.c_int32),
        ("error_code", C.c_int32),
        ("device_id", C.c_int32),
        ("hostname", C.c_char * 256),
        ("data_size", C.c_size_t),
        ("tensor_dim", C.c_size_t),
        ("current_offset", C.c_size_t),
        ("last_valid_offset", C.c_size_t),
        ("buffer_size", C.c_size_t),
        ("ipc_handle", C.c_ubyte * 64),
        ("tensor_shape", C.c_int64 * MAX_DIM),
    ]


# name -> (restype, argtypes); also the list of symbols the header declares.
_SIGNATURES = {
    "bikv_abi_version": (C.c_int, []),
    "bikv_last_error": (C.c_char_p, []),
    "bikv_init": (C.c_int, [C.c_int]),
    "bikv_check_status": (C.c_int, [C.c_int, C.c_void_p, C.POINTER(C.c_uint32)]),
    "bikv_set_tuning": (C.c_int, [C.c_char_p, C.c_int64]),
    "bikv_reset_tuning": (None, []),
    "bikv_find_duplicate": (C.c_int, [C.POINTER(C.c_int64), C.c_int64, C.POINTER(C.c_int64)]),
    "bikv_copy_runs": (C.c_int, [C.c_void_p, C.c_int64, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p,
                                 C.c_int64, C.c_int64, C.c_int64, C.c_void_p]),
    "bikv_copy_runs_ragged": (C.c_int, [C.c_void_p, C.c_int64, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p,
                                        C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_void_p]),
    "bikv_producer_copy_tokens": (C.c_int, [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p,
                                            C.c_int64, C.c_int64, C.c_int64, C.POINTER(TensorDimsC),
                                            C.c_int64, C.c_int32, C.c_void_p]),
    "bikv_pool_create": (C.c_int, [C.POINTER(PoolDesc), C.POINTER(C.c_void_p)]),
    "bikv_pool_destroy": (C.c_int, [C.c_void_p]),
    "bikv_gather_pages": (C.c_int, [C.c_void_p, C.POINTER(PageBatchDesc), C.c_void_p, C.c_int64,
                                    C.c_void_p, C.c_int64, C.c_void_p]),
    "bikv_scatter_pages": (C.c_int, [C.c_void_p, C.POINTER(PageBatchDesc), C.c_void_p, C.c_int64,
                                     C.c_void_p, C.c_int64, C.c_void_p]),
    "bikv_stager_create": (C.c_int, [C.c_int, C.c_int64, C.c_int32, C.c_int32, C.POINTER(C.c_void_p)]),
    "bikv_stager_wait": (C.c_int, [C.c_void_p, C.POINTER(StageStats)]),
    "bikv_stager_trace": (C.c_int, [C.c_void_p, C.c_int64]),
    "bikv_stager_trace_read": (C.c_int64, [C.c_void_p, C.POINTER(TraceStep), C.c_int64]),
    "bikv_gather_to_host_async": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(PageBatchDesc),
                                            C.POINTER(C.c_int64), C.c_int64, C.c_int32, C.c_void_p,
                                            C.c_int64, C.c_void_p, C.c_int64, C.c_int32, C.c_void_p]),
    "bikv_scatter_from_host_async": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(PageBatchDesc),
                                               C.POINTER(C.c_int64), C.c_int64, C.c_int32, C.c_void_p,
                                               C.c_int64, C.c_void_p, C.c_int64, C.c_int32, C.c_void_p]),
    "bikv_stager_destroy": (C.c_int, [C.c_void_p]),
    "bikv_gather_to_host": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(PageBatchDesc),
                                      C.POINTER(C.c_int64), C.c_int64, C.c_int32, C.c_void_p,
                                      C.c_int64, C.c_void_p, C.c_int64, C.c_int32, C.POINTER(StageStats)]),
    "bikv_scatter_from_host": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(PageBatchDesc),
                                         C.POINTER(C.c_int64), C.c_int64, C.c_int32, C.c_void_p,
                                         C.c_int64, C.c_void_p, C.c_int64, C.c_int32, C.POINTER(StageStats)]),
    "bikv_gather_to_host_noalloc": (C.c_int, [C.c_void_p, C.POINTER(PageBatchDesc), C.POINTER(C.c_int64), C.c_int64,
                                              C.c_int32, C.c_void_p, C.c_int64, C.c_void_p, C.c_int64, C.c_void_p]),
    "bikv_nhd_create": (C.c_int, [C.POINTER(NHDDesc), C.POINTER(C.c_void_p)]),
    "bikv_nhd_destroy": (C.c_int, [C.c_void_p]),
    "bikv_nhd_load_token_major": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p,
                                            C.c_int64, C.c_void_p]),
    "bikv_nhd_store_token_major": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p,
                                             C.c_int64, C.c_void_p]),
    "bikv_plan_chunks": (C.c_int64, [C.POINTER(C.c_int64), C.c_int64, C.c_int32, C.c_int32, C.c_int64,
                                     C.POINTER(C.c_int64), C.c_int64]),
    "bikv_d2h_copy": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64,
                                C.POINTER(C.c_double)]),
    "bikv_h2d_copy": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64,
                                C.POINTER(C.c_double)]),
    "bikv_device_alloc": (C.c_int, [C.c_int, C.c_int64, C.c_int32, C.POINTER(C.c_void_p)]),
    "bikv_device_alloc_bounded": (C.c_int, [C.c_int, C.c_int64, C.c_int32, C.c_int64, C.POINTER(C.c_void_p)]),
    "bikv_device_free": (C.c_int, [C.c_void_p]),
    "bikv_device_alloc_info": (C.c_int, [C.c_void_p, C.POINTER(AllocInfo)]),
    "bikv_torch_alloc": (C.c_void_p, [C.c_int64, C.c_int, C.c_void_p]),
    "bikv_torch_free": (None, [C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]),
    "bikv_host_alloc": (C.c_int, [C.c_int64, C.POINTER(C.c_void_p)]),
    "bikv_host_free": (C.c_int, [C.c_void_p]),
    "bikv_consumer_init": (C.c_int, [C.c_int, C.c_char_p, C.c_size_t]),
    "bikv_producer_init": (C.c_int, [C.c_int, C.c_char_p]),
    "bikv_producer_reserve": (C.c_int, [C.c_size_t, C.POINTER(C.c_void_p)]),
    "bikv_producer_publish": (C.c_int, [C.POINTER(C.c_int64), C.c_size_t, C.c_int32, C.c_void_p]),
    "bikv_producer_cancel": (C.c_int, []),
    "bikv_producer_set_backpressure": (C.c_int, [C.c_int, C.c_int64]),
    "bikv_consumer_release": (C.c_int, []),
    "bikv_producer_cleanup": (None, []),
    "bikv_consumer_cleanup": (None, []),
    "bikv_producer_copy_pages": (C.c_int, [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int64,
                                           C.c_int64, C.POINTER(TensorDimsC), C.c_int64, C.c_int32,
                                           C.c_void_p]),
    "bikv_producer_send": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_int64), C.c_size_t,
                                     C.c_int32, C.c_void_p]),
    "bikv_consumer_receive": (C.c_int, [C.c_int64, C.POINTER(C.c_void_p), C.POINTER(C.c_int64),
                                        C.POINTER(C.c_size_t), C.POINTER(C.c_size_t),
                                        C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "bikv_producer_control": (C.POINTER(SharedControl), []),
    "bikv_consumer_control": (C.POINTER(SharedControl), []),
    "bikv_consumer_buffer": (C.c_void_p, []),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib = None


def load():
    """Returns the loaded library; raises RuntimeError if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP library has not been built. Run "
            "`make -C bi-kv_amd/csrc` (or `python -c 'import __graft_entry__ as g; g.build()'`). "
            "There is no CPU fallback for this path."
        )
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here means header and library disagree
        fn.restype = res
        fn.argtypes = args
    got = lib.bikv_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError(f"libbikv_pagecopy.so has ABI version {got}, binding expects {ABI_VERSION}")
    _lib = lib
    return lib


def last_error():
    return load().bikv_last_error().decode("utf-8", "replace")


def check(rc):
    """Raises RuntimeError carrying the library's message when rc is a failure code."""
    if rc < 0:
        raise RuntimeError(last_error() or f"libbikv_pagecopy error {rc}")
    return rc


def set_tuning(**kw):
    lib = load()
    for k, v in kw.items():
        check(lib.bikv_set_tuning(k.encode(), int(v)))


def reset_tuning():
    """Every launch knob back to its default."""
    load().bikv_reset_tuning()


def require_unique(ids, what="page id"):
    """Raises RuntimeError naming the first repeated id of `ids` (any integer sequence or array on the
    host). The destinations of a scatter must be unique: two runs of one launch that write the same
    place race, as they do in the reference's kernel (copy_kernel.cu:29-35)."""
    import numpy as np
    arr = np.ascontiguousarray(np.asarray(ids, dtype=np.int64).reshape(-1))
    rc = load().bikv_find_duplicate(arr.ctypes.data_as(C.POINTER(C.c_int64)), arr.size, None)
    if rc < 0:
        raise RuntimeError(f"{what}: {last_error()}")
