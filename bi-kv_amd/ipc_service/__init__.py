"""`ipc_service` — drop-in for Bi-KV's pybind module of the same name, backed by libbikv_pagecopy.so.

Same names, argument order and error behaviour as the reference's module definition
(Bi-KV/SharedMemory/CUDA_Shared/ipc_service.cpp:240-257), so that
`import ipc_service` in Bi-KV/DistributedStorage/kvcache.py:26, Bi-KV/Worker/Worker.py:21 and the
two scripts test_page_ipc.py / test_zero_copy.py resolves to this package when `bi-kv_amd/` is on
sys.path:

    TensorDims                                   (ipc_wrapper.h:41-47)
    producer_init(device_id, shm_name)           consumer_init(device_id, shm_name, buffer_size)
    producer_send(tensor)                        consumer_receive() -> Tensor
    producer_cleanup()                           consumer_cleanup()
    producer_copy_pages(cache_data, src_offsets, dest_offsets, page_size, dims)
    producer_zero_copy_pages(cpu_data, page_indices, dest_offsets, page_size, dims)
    cuda_producer_copy_pages(...)                # exported by the reference but takes raw C++ pointers

Failures raise RuntimeError, as the reference's std::runtime_error / TORCH_CHECK do.

Differences a caller can observe (all extensions; fp16 callers see the reference's behaviour):
  * any dtype is accepted for the page copy; ring space is sized with the tensor's real element size
    (the reference sizes with sizeof(half) whatever the dtype, copy_kernel.cu:84) and the dtype is
    published so consumer_receive returns it (the reference always returns float16,
    ipc_service.cpp:157);
  * a batch larger than the whole ring raises instead of overrunning the buffer;
  * offsets that would leave the source tensor or the ring raise instead of faulting the GPU;
  * consumer_receive(timeout_ms=...) may be given a timeout (default: wait forever, as the reference);
  * producer_copy_tokens, producer_set_backpressure and consumer_release are additions (see each).
"""
import ctypes as C

import torch

from bikv_pagecopy import _lib

__all__ = [
    "TensorDims", "producer_init", "producer_send", "producer_cleanup", "consumer_init",
    "consumer_receive", "consumer_cleanup", "producer_copy_pages", "cuda_producer_copy_pages",
    "producer_zero_copy_pages", "producer_copy_tokens", "producer_set_backpressure", "consumer_release",
    "producer_reserve", "producer_publish", "producer_cancel",
]

# dtype codes carried in the control block's first spare int (0 = float16, what a reference
# producer leaves there).
_DTYPES = [torch.float16, torch.bfloat16, torch.float32, torch.float64, torch.uint8, torch.int8,
           torch.int16, torch.int32, torch.int64]
for _name in ("float8_e4m3fn", "float8_e5m2", "float8_e4m3fnuz", "float8_e5m2fnuz"):
    if hasattr(torch, _name):
        _DTYPES.append(getattr(torch, _name))
_CODE_OF = {dt: i for i, dt in enumerate(_DTYPES)}


class TensorDims:
    """ipc_wrapper.h:41-47 — five read/write ints, no-argument constructor."""

    __slots__ = ("total_tokens", "head_size", "num_kv_heads", "num_layers", "kv_pair")

    def __init__(self):
        self.total_tokens = 0
        self.head_size = 0
        self.num_kv_heads = 0
        self.num_layers = 0
        self.kv_pair = 0

    def _c(self):
        return _lib.TensorDimsC(int(self.total_tokens), int(self.head_size), int(self.num_kv_heads),
                                int(self.num_layers), int(self.kv_pair))


def _name(shm_name):
    return shm_name if isinstance(shm_name, bytes) else str(shm_name).encode()


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def consumer_init(device_id, shm_name, buffer_size):
    _lib.check(_lib.load().bikv_consumer_init(int(device_id), _name(shm_name), int(buffer_size)))


def producer_init(device_id, shm_name):
    _lib.check(_lib.load().bikv_producer_init(int(device_id), _name(shm_name)))


def producer_cleanup():
    _lib.load().bikv_producer_cleanup()


def consumer_cleanup():
    _lib.load().bikv_consumer_cleanup()


def producer_reserve(nbytes):
    """Not in the reference's module. Reserves `nbytes` of the consumer's ring (the reference's wrap
    rule, copy_kernel.cu:87-89) and returns them as a uint8 device tensor that the caller fills itself,
    e.g. as the staging image of PagedKVPool.gather; producer_publish then hands it to the consumer."""
    ptr = C.c_void_p()
    with torch.cuda.device(_producer_device()):
        _lib.check(_lib.load().bikv_producer_reserve(int(nbytes), C.byref(ptr)))
    device = torch.device("cuda", _producer_device())
    if nbytes == 0:
        return torch.empty(0, dtype=torch.uint8, device=device)
    return torch.as_tensor(_RingWindow(ptr.value, int(nbytes)), device=device)


def producer_publish(shape, dtype=torch.float16):
    """Publishes the reserved bytes as a tensor of `shape` (at most 5 dimensions) and `dtype`; waits for
    the current stream first and raises, publishing nothing, if a kernel writing the window skipped
    out-of-range work."""
    shape = tuple(int(x) for x in shape)
    if len(shape) > _lib.MAX_DIM:
        raise RuntimeError(f"Tensor must have at most {_lib.MAX_DIM} dimensions")
    if dtype not in _CODE_OF:
        raise RuntimeError(f"unsupported dtype {dtype}")
    arr = (C.c_int64 * _lib.MAX_DIM)(*shape)
    with torch.cuda.device(_producer_device()):
        _lib.check(_lib.load().bikv_producer_publish(arr, len(shape), _CODE_OF[dtype], _stream()))


def producer_cancel():
    """Not in the reference's module. Gives up a reserved window without publishing it. While a window
    is reserved every other producer call raises: it would be handed the same ring bytes."""
    _lib.check(_lib.load().bikv_producer_cancel())


def producer_set_backpressure(enabled, timeout_ms=-1):
    """Not in the reference's module. When enabled, a producer call that would overwrite a tensor the
    consumer has not released yet blocks (RuntimeError after timeout_ms); the consumer must then call
    consumer_release() once per received tensor, in order. Uses SharedControl.sem_complete, which the
    reference declares (ipc_wrapper.h:16) and never posts or waits on."""
    _lib.check(_lib.load().bikv_producer_set_backpressure(1 if enabled else 0, int(timeout_ms)))


def consumer_release():
    """Tells a back-pressured producer that the oldest tensor handed out by consumer_receive is no
    longer needed."""
    _lib.check(_lib.load().bikv_consumer_release())


def _producer_device():
    ctrl = _lib.load().bikv_producer_control()
    if not ctrl:
        raise RuntimeError("producer is not initialised")
    return ctrl.contents.device_id


def _check_offsets(name, t):
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be on CUDA")
    if t.dtype != torch.int64 or t.dim() != 1 or not t.is_contiguous():
        raise RuntimeError(f"{name} must be a contiguous 1-D int64 tensor")


def _copy_pages(data, src_offsets, dest_offsets, page_size, dims):
    if src_offsets.numel() != dest_offsets.numel():
        raise RuntimeError("src_offsets and dest_offsets differ in length")
    if data.dtype not in _CODE_OF:
        raise RuntimeError(f"unsupported dtype {data.dtype}")
    d = dims._c()
    es = data.element_size()
    with torch.cuda.device(_producer_device()):
        _lib.check(_lib.load().bikv_producer_copy_pages(
            data.data_ptr(), data.numel() * es, src_offsets.data_ptr(), dest_offsets.data_ptr(),
            src_offsets.numel(), int(page_size), C.byref(d), es, _CODE_OF[data.dtype], _stream()))


def producer_copy_tokens(data, src_token_offsets, dest_token_offsets, run_tokens, page_size, dims):
    """Not in the reference's module: the packed transfer done right. Offsets and `run_tokens`
    are in TOKENS, the unit kvcache.py:161-196 computes them in; run i copies run_tokens[i] <=
    page_size tokens, so the packed destinations of partial last pages (kvcache.py:169-174) do not
    overlap. `dims.total_tokens` must hold the sum of run_tokens (the host already has it from
    building the offsets); the published shape is [total_tokens, head, kv_heads, layers, kv].
    `data` may be a device tensor or a pinned host tensor (read over the link)."""
    if not data.is_cuda and not data.is_pinned():
        raise RuntimeError("CPU data must be pinned memory")
    if not data.is_contiguous():
        raise RuntimeError("Cache data must be contiguous")
    for name, t in (("src_offsets", src_token_offsets), ("dest_offsets", dest_token_offsets),
                    ("run_tokens", run_tokens)):
        _check_offsets(name, t)
    if not (src_token_offsets.numel() == dest_token_offsets.numel() == run_tokens.numel()):
        raise RuntimeError("offset and length tables differ in length")
    if data.dtype not in _CODE_OF:
        raise RuntimeError(f"unsupported dtype {data.dtype}")
    d = dims._c()
    es = data.element_size()
    with torch.cuda.device(_producer_device()):
        _lib.check(_lib.load().bikv_producer_copy_tokens(
            data.data_ptr(), data.numel() * es, src_token_offsets.data_ptr(), dest_token_offsets.data_ptr(),
            run_tokens.data_ptr(), run_tokens.numel(), int(page_size), int(dims.total_tokens), C.byref(d), es,
            _CODE_OF[data.dtype], _stream()))


def producer_copy_pages(cache_data, src_offsets, dest_offsets, page_size, dims):
    """copy_kernel.cu:68-129. Offsets are element offsets into cache_data / the ring write window."""
    if not cache_data.is_cuda:
        raise RuntimeError("Cache data must be on CUDA")
    if not cache_data.is_contiguous():
        raise RuntimeError("Cache data must be contiguous")
    _check_offsets("src_offsets", src_offsets)
    _check_offsets("dest_offsets", dest_offsets)
    _copy_pages(cache_data, src_offsets, dest_offsets, page_size, dims)


def producer_zero_copy_pages(cpu_data, page_indices, dest_offsets, page_size, dims):
    """copy_kernel.cu:133-196. `page_indices` are used as ELEMENT offsets into cpu_data, exactly as
    the reference's kernel does (copy_kernel.cu:52)."""
    if cpu_data.is_cuda or not cpu_data.is_pinned():
        raise RuntimeError("CPU data must be pinned memory")
    if not cpu_data.is_contiguous():
        raise RuntimeError("CPU data must be contiguous")
    if not page_indices.is_cuda:
        raise RuntimeError("Page indices must be on CUDA")
    if not dest_offsets.is_cuda:
        raise RuntimeError("Dest offsets must be on CUDA")
    _check_offsets("page_indices", page_indices)
    _check_offsets("dest_offsets", dest_offsets)
    _copy_pages(cpu_data, page_indices, dest_offsets, page_size, dims)


def cuda_producer_copy_pages(cache_data, src_offsets, dest_offsets, ctrl, shm_ptr, page_size, dims):
    """Bound by the reference (ipc_service.cpp:255) with raw SharedControl*/void* parameters that no
    Python caller can supply; kept so the name resolves."""
    raise RuntimeError("cuda_producer_copy_pages takes raw C++ pointers; call producer_copy_pages")


def producer_send(tensor):
    """ipc_service.cpp:113-143: contiguous float16 CUDA tensor -> ring, shape published."""
    if not tensor.is_cuda:
        raise RuntimeError("Tensor must be on CUDA")
    if not tensor.is_contiguous():
        raise RuntimeError("Tensor must be contiguous")
    if tensor.dtype != torch.float16:
        raise RuntimeError("Tensor must be float16")
    if tensor.dim() > _lib.MAX_DIM:
        raise RuntimeError(f"Tensor must have at most {_lib.MAX_DIM} dimensions")
    shape = (C.c_int64 * _lib.MAX_DIM)(*tensor.shape)
    with torch.cuda.device(_producer_device()):
        _lib.check(_lib.load().bikv_producer_send(
            tensor.data_ptr(), tensor.numel() * tensor.element_size(), shape, tensor.dim(),
            _CODE_OF[tensor.dtype], _stream()))


class _RingWindow:
    """Exposes a span of the consumer's ring to torch without copying or owning it."""

    def __init__(self, ptr, nbytes):
        self.__cuda_array_interface__ = {
            "shape": (int(nbytes),), "typestr": "|u1", "data": (int(ptr), False), "version": 2,
            "strides": None,
        }


def consumer_receive(timeout_ms=-1):
    """ipc_service.cpp:146-168: waits for the producer, returns a non-owning view of the ring."""
    ptr = C.c_void_p()
    shape = (C.c_int64 * _lib.MAX_DIM)()
    ndim = C.c_size_t()
    nbytes = C.c_size_t()
    dev = C.c_int32()
    code = C.c_int32()
    _lib.check(_lib.load().bikv_consumer_receive(
        int(timeout_ms), C.byref(ptr), shape, C.byref(ndim), C.byref(nbytes), C.byref(dev), C.byref(code)))
    dims = tuple(int(shape[i]) for i in range(ndim.value))
    dtype = _DTYPES[code.value] if 0 <= code.value < len(_DTYPES) else torch.float16
    n = 1
    for s in dims:
        n *= s
    want = n * torch.empty((), dtype=dtype).element_size()
    device = torch.device("cuda", dev.value)
    if want == 0:
        return torch.empty(dims, dtype=dtype, device=device)
    raw = torch.as_tensor(_RingWindow(ptr.value, want), device=device)
    return raw.view(dtype).reshape(dims)
