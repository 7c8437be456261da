"""ctypes binding of the two shared libraries of the gfx950 DIOPI backend.

``libdiopirt_hip.so`` implements the caller side of the DIOPI runtime interface
(tensor accessors, stream, context-owned scratch); ``libdiopi_impl.so`` is the
operator library and resolves those callbacks against it at load time, exactly
as it would against a framework's own runtime.  This module plays the role of
``diopi_test/python/conformance/diopi_runtime.py`` of the reference (Tensor /
Context / Sizes / Dtype at diopi_runtime.py:72-365), with torch tensors as the
owners of device memory.

Nothing here computes: if the operator library cannot be loaded, importing the
functions raises; there is no fallback path.
"""
from __future__ import annotations

import ctypes
import enum
import os
import threading
from typing import Optional, Sequence

import torch

# the in-tree build; DIOPI_AMD_LIB_DIR points the package at another build of the same two libraries
_LIB_DIR = os.environ.get("DIOPI_AMD_LIB_DIR") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
RT_LIB_PATH = os.path.join(_LIB_DIR, "libdiopirt_hip.so")
IMPL_LIB_PATH = os.path.join(_LIB_DIR, "libdiopi_impl.so")


class diopiError(enum.IntEnum):
    """diopiError_t (include/diopi/diopirt.h)."""
    diopi_success = 0
    diopi_error_occurred = 1
    diopi_no_implement = 13
    diopi_force_fallback_to_cpu = 14
    diopi_dtype_not_supported = 1000


class Dtype(enum.IntEnum):
    """diopiDtype_t (include/diopi/diopirt.h)."""
    int8 = 0
    uint8 = 1
    int16 = 2
    uint16 = 3
    int32 = 4
    uint32 = 5
    int64 = 6
    uint64 = 7
    float16 = 8
    float32 = 9
    float64 = 10
    bool = 11
    bfloat16 = 12


class Device(enum.IntEnum):
    Host = 0
    AIChip = 1


_TORCH_TO_DTYPE = {
    torch.int8: Dtype.int8,
    torch.uint8: Dtype.uint8,
    torch.int16: Dtype.int16,
    torch.int32: Dtype.int32,
    torch.int64: Dtype.int64,
    torch.float16: Dtype.float16,
    torch.float32: Dtype.float32,
    torch.float64: Dtype.float64,
    torch.bool: Dtype.bool,
    torch.bfloat16: Dtype.bfloat16,
}


class _SizeStruct(ctypes.Structure):
    """diopiSize_t: a borrowed int64 array, passed by value."""
    _fields_ = [("data", ctypes.POINTER(ctypes.c_int64)), ("len", ctypes.c_int64)]


class Sizes:
    """Owner of the int64 storage behind a diopiSize_t (reference: diopi_runtime.py Sizes)."""

    def __init__(self, values: Sequence[int]):
        self.values = [int(v) for v in values]
        self._array = (ctypes.c_int64 * max(len(self.values), 1))(*self.values)
        self.c = _SizeStruct(ctypes.cast(self._array, ctypes.POINTER(ctypes.c_int64)), len(self.values))


class DiopiException(Exception):
    """A call returned a failure code; the text is diopiGetLastErrorString()."""


class FunctionNotImplementedError(DiopiException):
    """The call returned diopiNoImplement (13): the conformance harness skips such cases."""


_libs_lock = threading.Lock()
_libs = None


class _Libs:
    def __init__(self):
        if not (os.path.exists(RT_LIB_PATH) and os.path.exists(IMPL_LIB_PATH)):
            raise ImportError(
                f"the HIP libraries are not built ({RT_LIB_PATH}, {IMPL_LIB_PATH}); run `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C diopi_amd/csrc`")
        # the operator library imports the diopirt callbacks: they must be globally visible first
        self.rt = ctypes.CDLL(RT_LIB_PATH, mode=ctypes.RTLD_GLOBAL)
        self.impl = ctypes.CDLL(IMPL_LIB_PATH, mode=ctypes.RTLD_GLOBAL)
        rt, impl = self.rt, self.impl
        vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
        rt.diopirtDeviceCount.restype = i32
        rt.diopirtDeviceClockKHz.restype, rt.diopirtDeviceClockKHz.argtypes = i32, [i32]
        rt.diopirtDeviceComputeUnits.restype, rt.diopirtDeviceComputeUnits.argtypes = i32, [i32]
        rt.diopirtContextCreate.restype = vp
        rt.diopirtContextCreate.argtypes = [vp]
        rt.diopirtContextDestroy.argtypes = [vp]
        rt.diopirtContextClearTensors.argtypes = [vp]
        rt.diopirtContextSynchronize.argtypes = [vp]
        rt.diopirtContextSynchronize.restype = i32
        for name in ("diopirtContextScratchInUse", "diopirtContextScratchPeak", "diopirtContextMallocCount"):
            getattr(rt, name).argtypes = [vp]
            getattr(rt, name).restype = i64
        rt.diopirtTensorWrap.restype = vp
        rt.diopirtTensorWrap.argtypes = [vp, ctypes.POINTER(i64), ctypes.POINTER(i64), i64, i32, i32]
        rt.diopirtTensorDestroy.argtypes = [vp]
        rt.diopirtEventCreate.restype = vp
        rt.diopirtEventDestroy.argtypes = [vp]
        rt.diopirtEventRecord.argtypes = [vp, vp]
        rt.diopirtEventRecord.restype = i32
        rt.diopirtEventElapsedMs.argtypes = [vp, vp]
        rt.diopirtEventElapsedMs.restype = ctypes.c_float
        rt.diopirtItemsize.argtypes = [i32]
        rt.diopirtItemsize.restype = i64
        # the device hooks of the reference's harness (conform_test.h:28-43)
        u64 = ctypes.c_uint64
        rt.device_malloc.restype, rt.device_malloc.argtypes = vp, [u64]
        rt.device_free.restype, rt.device_free.argtypes = None, [vp]
        for name in ("device_memcpy_h2d_async", "device_memcpy_d2h_async", "device_memcpy_d2d_async"):
            getattr(rt, name).restype, getattr(rt, name).argtypes = i32, [vp, vp, vp, u64]
        rt.device_make_stream.restype, rt.device_make_stream.argtypes = i32, [ctypes.POINTER(vp)]
        rt.device_destroy_stream.restype, rt.device_destroy_stream.argtypes = i32, [vp]
        rt.device_synchronize_stream.restype, rt.device_synchronize_stream.argtypes = i32, [vp]
        rt.initLibrary.restype, rt.initLibrary.argtypes = i32, []
        rt.finalizeLibrary.restype, rt.finalizeLibrary.argtypes = i32, []
        rt.buildGeneratorState.restype, rt.buildGeneratorState.argtypes = i32, [vp, vp]
        rt.diopiGetTensorNumel.restype, rt.diopiGetTensorNumel.argtypes = i32, [vp, ctypes.POINTER(i64)]
        rt.diopiGetTensorDtype.restype, rt.diopiGetTensorDtype.argtypes = i32, [vp, ctypes.POINTER(i32)]
        rt.diopiGetTensorDevice.restype, rt.diopiGetTensorDevice.argtypes = i32, [vp, ctypes.POINTER(i32)]

        for name in ("diopiGetVendorName", "diopiGetImplVersion", "diopiGetLastErrorString"):
            getattr(impl, name).restype = ctypes.c_char_p
            getattr(impl, name).argtypes = []
        b = ctypes.c_bool
        impl.diopiRotaryEmbedding.argtypes = [vp, vp, vp, vp, vp, b, b]
        impl.diopiRotaryEmbeddingV2.argtypes = [vp, vp, vp, vp, vp, i64]
        impl.diopiApplyPenalty.argtypes = [vp, vp, vp, vp, vp, vp, vp, i32]
        impl.diopiApplyPenaltyV2.argtypes = [vp, vp, vp, vp, vp, vp, vp]
        impl.diopiRMSNorm.argtypes = [vp, vp, vp, vp, _SizeStruct, vp, vp, ctypes.c_double]
        impl.diopiRMSNormBackward.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, _SizeStruct, ctypes.c_double]
        impl.diopiDestIndexCopyKV.argtypes = [vp, vp, vp, vp]
        impl.diopiTokenAttentionInference.argtypes = [vp, vp, vp, vp, vp, vp, vp, i32]
        impl.diopiTokenSoftmaxReduceVInference.argtypes = [vp, vp, vp, vp, vp, vp, vp, i32, i32]
        impl.diopiContextAttentionInference.argtypes = [vp, vp, vp, vp, vp, vp, vp, i32]
        impl.diopiContextAttentionInferenceNoAlloc.argtypes = [vp, vp, vp, vp, vp, vp, vp, i32]
        impl.diopiFlashAttentionVarLen.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, ctypes.c_float, ctypes.c_float, ctypes.c_bool,
                                                   i32, i32]
        impl.diopiFlashAttention.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, ctypes.c_float, ctypes.c_float, ctypes.c_bool, i32, i32]
        i64, dbl = ctypes.c_int64, ctypes.c_double
        impl.diopiMultiHeadAttention.argtypes = [vp, vp, vp, vp, dbl, ctypes.c_bool, ctypes.c_bool, dbl, vp, vp, vp, vp]
        impl.diopiMultiHeadAttentionVarLen.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, dbl, ctypes.c_bool, ctypes.c_bool, dbl, vp, vp, vp, vp]
        impl.diopiPagedAttention.argtypes = [vp, vp, vp, vp, vp, vp, _SizeStruct, i64, i64, i64, vp, i64]
        impl.diopiPromptFlashAttention.argtypes = [vp, vp, vp, vp, vp, vp, _SizeStruct, i64, i64, i64, i64]
        impl.diopiRootMeanSquareNormInp.argtypes = [vp, vp, vp, ctypes.c_float]
        impl.diopiFusedAddRootMeanSquareNormInp.argtypes = [vp, vp, vp, vp, vp, ctypes.c_float]
        impl.diopiFusedDecoderAttentionInp.argtypes = [vp, vp, vp, vp, vp, ctypes.POINTER(i64), i64, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64,
                                                       ctypes.c_float]
        for name in OPERATOR_SYMBOLS:
            getattr(impl, name).restype = i32


# Every symbol include/diopi/functions.h, functions_ext.h and functions_lmdeploy.h declare.
OPERATOR_SYMBOLS = (
    "diopiRotaryEmbedding",
    "diopiRotaryEmbeddingV2",
    "diopiApplyPenalty",
    "diopiApplyPenaltyV2",
    "diopiRMSNorm",
    "diopiRMSNormBackward",
    "diopiDestIndexCopyKV",
    "diopiTokenAttentionInference",
    "diopiTokenSoftmaxReduceVInference",
    "diopiContextAttentionInference",
    "diopiContextAttentionInferenceNoAlloc",
    "diopiFlashAttentionVarLen",
    "diopiFlashAttention",
    "diopiMultiHeadAttention",
    "diopiMultiHeadAttentionVarLen",
    "diopiPagedAttention",
    "diopiPromptFlashAttention",
    "diopiRootMeanSquareNormInp",
    "diopiFusedAddRootMeanSquareNormInp",
    "diopiFusedDecoderAttentionInp",
)
INFO_SYMBOLS = ("diopiGetVendorName", "diopiGetImplVersion", "diopiGetLastErrorString")


def libs() -> _Libs:
    global _libs
    with _libs_lock:
        if _libs is None:
            _libs = _Libs()
        return _libs


def device_count() -> int:
    return int(libs().rt.diopirtDeviceCount())


def get_last_error_string() -> str:
    return libs().impl.diopiGetLastErrorString().decode("utf-8", "replace")


def check_returncode(ret: int, call: str = "") -> None:
    """Same policy as diopi_functions.py:65-79 of the reference."""
    if ret == diopiError.diopi_success:
        return
    msg = f"{call} returned {ret}: {get_last_error_string()}"
    if ret == diopiError.diopi_no_implement:
        raise FunctionNotImplementedError(msg)
    raise DiopiException(msg)


class Context:
    """A diopiContext: one stream plus the scratch tensors handed out on it."""

    def __init__(self, stream: Optional[torch.cuda.Stream] = None, own_stream: bool = False):
        self._rt = libs().rt
        self.torch_stream = stream
        if stream is None and not own_stream and torch.cuda.is_available():
            self.torch_stream = torch.cuda.Stream()
        handle = self.torch_stream.cuda_stream if self.torch_stream is not None else None
        self.handle = ctypes.c_void_p(self._rt.diopirtContextCreate(ctypes.c_void_p(handle)))

    def synchronize(self) -> None:
        ret = self._rt.diopirtContextSynchronize(self.handle)
        if ret != 0:
            raise DiopiException("stream synchronisation failed")

    def clear_tensors(self) -> None:
        self._rt.diopirtContextClearTensors(self.handle)

    @property
    def scratch_peak(self) -> int:
        return int(self._rt.diopirtContextScratchPeak(self.handle))

    @property
    def malloc_count(self) -> int:
        return int(self._rt.diopirtContextMallocCount(self.handle))

    def close(self) -> None:
        if self.handle:
            self._rt.diopirtContextDestroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Tensor:
    """A diopiTensor handle over the memory of a torch tensor (which it keeps alive)."""

    def __init__(self, t: torch.Tensor):
        if t.dtype not in _TORCH_TO_DTYPE:
            raise TypeError(f"unsupported dtype {t.dtype}")
        self.torch = t
        self._rt = libs().rt
        nd = t.dim()
        shape = (ctypes.c_int64 * max(nd, 1))(*t.shape)
        stride = (ctypes.c_int64 * max(nd, 1))(*t.stride())
        device = Device.AIChip if t.is_cuda else Device.Host
        ptr = t.data_ptr() if t.numel() > 0 else 0
        self.handle = ctypes.c_void_p(
            self._rt.diopirtTensorWrap(ctypes.c_void_p(ptr), shape, stride, nd, int(_TORCH_TO_DTYPE[t.dtype]), int(device)))
        if not self.handle:
            raise DiopiException("diopirtTensorWrap failed")

    def __del__(self):
        try:
            if self.handle:
                self._rt.diopirtTensorDestroy(self.handle)
                self.handle = None
        except Exception:
            pass


def as_handle(t):
    """None -> NULL handle (optional tensors), Tensor -> its handle."""
    return None if t is None else t.handle


class Event:
    """A HIP event recorded on a context's stream."""

    def __init__(self):
        self._rt = libs().rt
        self.handle = ctypes.c_void_p(self._rt.diopirtEventCreate())
        if not self.handle:
            raise DiopiException("hipEventCreate failed")

    def record(self, ctx: Context) -> None:
        if self._rt.diopirtEventRecord(self.handle, ctx.handle) != 0:
            raise DiopiException("hipEventRecord failed")

    def elapsed_ms(self, stop: "Event") -> float:
        ms = float(self._rt.diopirtEventElapsedMs(self.handle, stop.handle))
        if ms < 0:
            raise DiopiException("hipEventElapsedTime failed")
        return ms

    def __del__(self):
        try:
            if self.handle:
                self._rt.diopirtEventDestroy(self.handle)
                self.handle = None
        except Exception:
            pass


_default_ctx = None


def default_context() -> Context:
    """Created on first use (reference: diopi_runtime.py:235 creates it at import)."""
    global _default_ctx
    if _default_ctx is None:
        _default_ctx = Context()
    return _default_ctx
