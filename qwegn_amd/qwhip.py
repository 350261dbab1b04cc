"""ctypes binding of libqwhip's C ABI (include/qwhip.h), used by the tests and the benchmark.

It binds the exported symbols 1:1 and adds nothing but buffer bookkeeping: no compute happens
on the host and there is no fallback - a missing library or a failing call raises.
"""
from __future__ import annotations

import ctypes as C
import pathlib

import numpy as np

LIB_PATH = pathlib.Path(__file__).resolve().parent / "lib" / "libqwhip.so"

OK = 0
E_BAD_WEIGHTS, E_BAD_SHAPE, E_BAD_GEOMETRY, E_BLOCKED, E_KERNEL_MISSING, E_DEVICE, E_BASIS, E_NULL, E_ALLOC = range(1, 10)
F32, F16, BF16, I32 = 0, 1, 2, 3
KIND_HQ4_G32_M5, KIND_ROTATED_HQ, KIND_NATIVE_AFFINE = 0, 1, 2
X_PREROTATED = 1
GEMV_ROW_INVARIANT = 2
MOE_REUSE_EXPERTS = 4


class QwhipError(RuntimeError):
    def __init__(self, status: int, name: str, message: str):
        super().__init__(f"qwhip status {status} ({name}): {message}")
        self.status = status
        self.name = name


class WeightView(C.Structure):
    _fields_ = [("blocks", C.c_void_p), ("bytes", C.c_uint64), ("n", C.c_uint32), ("k", C.c_uint32),
                ("kind", C.c_uint32), ("bits", C.c_uint32), ("group", C.c_uint32)]


class Caps(C.Structure):
    _fields_ = [("name", C.c_char * 64), ("arch", C.c_char * 32), ("compute_units", C.c_uint32),
                ("wavefront", C.c_uint32), ("lds_bytes", C.c_uint32), ("l2_bytes", C.c_uint32),
                ("hbm_bytes", C.c_uint64), ("clock_khz", C.c_uint32), ("has_mfma_f16", C.c_uint32)]


_P = C.c_void_p
_U32 = C.c_uint32
_U64 = C.c_uint64
_WV = C.POINTER(WeightView)

# name -> (restype, argtypes); one entry per declaration in include/qwhip.h
SIGNATURES = {
    "qwhip_device_create": (C.c_int32, [C.c_int32, C.POINTER(_P)]),
    "qwhip_device_destroy": (C.c_int32, [_P]),
    "qwhip_device_caps": (C.c_int32, [_P, C.POINTER(Caps)]),
    "qwhip_stream_create": (C.c_int32, [_P, C.POINTER(_P)]),
    "qwhip_stream_destroy": (C.c_int32, [_P]),
    "qwhip_stream_sync": (C.c_int32, [_P]),
    "qwhip_stream_native": (_P, [_P]),
    "qwhip_malloc": (C.c_int32, [_P, C.c_size_t, C.POINTER(_P)]),
    "qwhip_free": (C.c_int32, [_P, _P]),
    "qwhip_memcpy_h2d": (C.c_int32, [_P, _P, _P, C.c_size_t]),
    "qwhip_memcpy_d2h": (C.c_int32, [_P, _P, _P, C.c_size_t]),
    "qwhip_memcpy_d2d": (C.c_int32, [_P, _P, _P, C.c_size_t]),
    "qwhip_fill_u32": (C.c_int32, [_P, _P, _U32, C.c_size_t]),
    "qwhip_plane_checksum": (C.c_int32, [_P, _P, C.c_size_t, _P]),
    "qwhip_plane_checksum_rows": (C.c_int32, [_P, _P, C.c_uint32, C.c_uint32, _P]),
    "qwhip_event_create": (C.c_int32, [_P, C.POINTER(_P)]),
    "qwhip_event_destroy": (C.c_int32, [_P]),
    "qwhip_event_record": (C.c_int32, [_P, _P]),
    "qwhip_event_elapsed_ms": (C.c_int32, [_P, _P, C.POINTER(C.c_float)]),
    "qwhip_kernel_lookup": (C.c_int32, [C.c_char_p, C.POINTER(C.c_char_p)]),
    "qwhip_last_error": (C.c_char_p, []),
    "qwhip_status_name": (C.c_char_p, [C.c_int32]),
    "qwhip_block_bytes": (_U32, [_U32, _U32, _U32]),
    "qwhip_weight_view_validate": (C.c_int32, [_WV]),
    "qwhip_fwht32": (C.c_int32, [_P, _P, _U32, _P, _U64]),
    "qwhip_cast_f32_to_f16": (C.c_int32, [_P, _P, _P, _U64]),
    "qwhip_swiglu_fwht": (C.c_int32, [_P, _P, _U32, _P, _U32, _U32, _U32]),
    "qwhip_dequant_f16": (C.c_int32, [_P, _WV, _P]),
    "qwhip_gemv": (C.c_int32, [_P, _WV, _P, _U32, _U32, _U32, _P, _P]),
    "qwhip_gemv_silu_pair": (C.c_int32, [_P, _WV, _P, _U32, _U32, _U32, _U32, _P]),
    "qwhip_gemm": (C.c_int32, [_P, _WV, _P, _U32, _U32, _U32, _P, _U32, _U32, _U32, _P, _U64]),
    "qwhip_gemm_noalloc": (C.c_int32, [_P, _WV, _P, _U32, _U32, _U32, _P, _U32, _U32, _U32]),
    "qwhip_gemm_noalloc_max_bytes": (_U64, []),
    "qwhip_moe_route": (C.c_int32, [_P, _P, _U32, _U32, _U32, _U32, C.c_float, _P, _P]),
    "qwhip_moe_route_ex": (C.c_int32, [_P, _P, _U32, _U32, _U32, _U32, C.c_float, _U32, _P, _P, _P, _P]),
    "qwhip_router_gemm": (C.c_int32, [_P, _P, _U32, _P, _U32, _U32, _U32, _U32, _P]),
    "qwhip_silu_mul_f32": (C.c_int32, [_P, _P, _P, _U32, _U32]),
    "qwhip_moe_bridge_f16_to_f32": (C.c_int32, [_P, _P, _P, _P, _U32, _U32]),
    "qwhip_latent_norm_h32_f32": (C.c_int32, [_P, _P, _P, _P, _P, _U32, _U32, C.c_float]),
    "qwhip_add_f32": (C.c_int32, [_P, _P, _P, _P, C.c_uint64]),
    "qwhip_embed_bf16_f32": (C.c_int32, [_P, _P, _U32, _U32, _P, _U32, _U32, _P]),
    "qwhip_embed_aq_f32": (C.c_int32, [_P, _P, _P, _U32, _U32, _P]),
    "qwhip_router_gemm_shared_gate": (C.c_int32, [_P, _P, _U32, _P, _U32, _U32, _U32, _U32, _P, _P, _P]),
    "qwhip_moe_max_tiles": (_U32, [_U32, _U32]),
    "qwhip_moe_group_pairs": (C.c_int32, [_P, _P, _U32, _U32, _U32, _P, _P, _P, _P, _P, _P, _P, _U32]),
    "qwhip_moe_grouped_gemm": (C.c_int32, [_P, _WV, _U32, _P, _U32, _U32, _P, _P, _P, _P, _P, _U32, _U32, _P, _U32, _U32]),
    "qwhip_gemm_swiglu": (C.c_int32, [_P, _WV, _P, _U32, _U32, _U32, _U32, _P, _U32, _U32, _P, C.c_size_t]),
    "qwhip_moe_grouped_gemm_swiglu": (C.c_int32, [_P, _WV, _U32, _P, _U32, _U32, _P, _P, _P, _P, _P, _U32, _U32, _U32, _P, _U32]),
    "qwhip_moe_combine": (C.c_int32, [_P, _P, _U32, _P, _P, _U32, _U32, _U32, _P, _P, _P, _U32]),
    "qwhip_moe_gateup_decode": (C.c_int32, [_P, _WV, _U32, _P, _U32, _U32, _P, _U32, _U32, _P]),
    "qwhip_moe_route_gateup_decode": (C.c_int32, [_P, _WV, _U32, _P, _U32, _U32, _P, _U32, _U32, _U32, C.c_float, _P, _P, _P]),
    "qwhip_moe_down_decode": (C.c_int32, [_P, _WV, _U32, _P, _P, _P, _U32, _U32, _P, _P, _P, _U32]),
    "qwhip_device_set_gated_activation": (C.c_int32, [_P, _U32, C.c_float, C.c_float]),
    "qwhip_moe_route_budget": (C.c_int32, [_P, _P, _P, _U32, _U32, _U32, _U32]),
    "qwhip_moe_latent_groups": (C.c_int32, [_P, _P, _P, _U32, _U32, _U32, _U32, _P, _P]),
    "qwhip_moe_routed_gemv": (C.c_int32, [_P, _WV, _U32, _P, _U32, _P, _P, _U32, _U32, _P, _U32]),
    "qwhip_moe_gateup_decode_rows": (C.c_int32, [_P, _WV, _U32, _P, _U32, _U32, _P, _P, _U32, _U32, _P]),
    "qwhip_moe_down_decode_groups": (C.c_int32, [_P, _WV, _U32, _P, _P, _P, _P, _U32, _U32, _U32, _P, _U32]),
    "qwhip_moe_compose_rows": (C.c_int32, [_P, _P, _U32, _P, _U32, _P, _P]),
    "qwhip_moe_combine_groups": (C.c_int32, [_P, _P, _U32, _P, _P, _P, _P, _U32, _U32, _U32, _U32, _U32, _P, _U32]),
    "qwhip_quantize_hq4_g32": (C.c_int32, [_P, _P, _U32, _U32, _U32, _U32, _P]),
    "qwhip_quantize_blocks": (C.c_int32, [_P, _P, _U32, _U32, _U32, _U32, _U32, _U32, _U32, _P]),
    "qwhip_quantize_hq8_planar": (C.c_int32, [_P, _P, _U32, _U32, _U32, _U32, _P, _P]),
    "qwhip_dequant_hq8_planar": (C.c_int32, [_P, _P, _P, _U32, _U32, _P]),
    "qwhip_head_argmax": (C.c_int32, [_P, _WV, _P, _U32, _U32, _U32, _P, _P]),
    "qwhip_argmax_f32": (C.c_int32, [_P, _P, _U32, _U32, _P]),
    "qwhip_argmax_f32_variational": (C.c_int32, [_P, _P, _U32, _U32, _P, _U32, C.c_float, C.c_float, _P]),
    "qwhip_f32_gemv": (C.c_int32, [_P, _P, _P, _U32, _U32, _U32, _U32, C.c_float, _P]),
    "qwhip_gemv_f32": (C.c_int32, [_P, _WV, _P, _U32, _U32, C.c_float, _P]),
    "qwhip_h32_f32": (C.c_int32, [_P, _P, _P, _U32, _U32]),
    "qwhip_rmsnorm": (C.c_int32, [_P, _P, _P, _P, _U32, _U32, C.c_float, _U32, _P]),
    "qwhip_repack_mlx_affine": (C.c_int32, [_P, _P, _P, _P, _U32, _U32, _U32, _U32, _U32, _P, _P]),
    "qwhip_repack_mlx_affine_switch_gate_up": (C.c_int32, [_P, _P, _P, _P, _P, _P, _P, _U32, _U32, _U32, _U32, _U32, _U32, _P, _P]),
}

_lib = None


def load() -> C.CDLL:
    """Loads libqwhip.so and binds every symbol; raises if the library or a symbol is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m qwegn_amd.build` (there is no CPU fallback)")
    lib = C.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(status: int) -> None:
    if status != OK:
        lib = load()
        raise QwhipError(status, lib.qwhip_status_name(status).decode(), lib.qwhip_last_error().decode())


NP_DTYPES = {F32: np.float32, F16: np.float16, BF16: np.uint16, I32: np.int32}


class Buffer:
    """A device allocation owned by the test or benchmark (stands for an arena region)."""

    def __init__(self, dev: "Device", nbytes: int):
        self.dev = dev
        self.nbytes = int(nbytes)
        p = _P()
        check(dev.lib.qwhip_malloc(dev.handle, self.nbytes, C.byref(p)))
        self.ptr = p.value

    def upload(self, arr: np.ndarray, stream: "Stream | None" = None) -> "Buffer":
        a = np.ascontiguousarray(arr)
        assert a.nbytes <= self.nbytes, (a.nbytes, self.nbytes)
        st = stream or self.dev.stream
        check(self.dev.lib.qwhip_memcpy_h2d(st.handle, self.ptr, a.ctypes.data, a.nbytes))
        return self

    def download(self, dtype, shape, stream: "Stream | None" = None) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes, (out.nbytes, self.nbytes)
        st = stream or self.dev.stream
        check(self.dev.lib.qwhip_memcpy_d2h(st.handle, out.ctypes.data, self.ptr, out.nbytes))
        return out

    def free(self) -> None:
        if self.ptr:
            check(self.dev.lib.qwhip_free(self.dev.handle, self.ptr))
            self.ptr = None


class Stream:
    def __init__(self, dev: "Device"):
        self.dev = dev
        h = _P()
        check(dev.lib.qwhip_stream_create(dev.handle, C.byref(h)))
        self.handle = h.value

    def sync(self) -> None:
        check(self.dev.lib.qwhip_stream_sync(self.handle))


class Event:
    def __init__(self, dev: "Device"):
        self.dev = dev
        h = _P()
        check(dev.lib.qwhip_event_create(dev.handle, C.byref(h)))
        self.handle = h.value

    def record(self, stream: Stream) -> None:
        check(self.dev.lib.qwhip_event_record(self.handle, stream.handle))

    def elapsed_ms(self, stop: "Event") -> float:
        ms = C.c_float()
        check(self.dev.lib.qwhip_event_elapsed_ms(self.handle, stop.handle, C.byref(ms)))
        return float(ms.value)


class Graph:
    """A HIP graph of the launches a callable puts on a stream (the library's launch doors only enqueue kernels: no
    allocation, no copy, no clear, so a chain of them can be captured), for callers whose steps are bound by launch
    latency.  capture() runs `fn` once under stream capture; launch() replays the recorded kernels with the arguments they
    were recorded with."""

    _hip = None

    @classmethod
    def _rt(cls) -> C.CDLL:
        if cls._hip is None:
            hip = C.CDLL("libamdhip64.so")
            hip.hipStreamBeginCapture.argtypes = [_P, C.c_int]
            hip.hipStreamEndCapture.argtypes = [_P, C.POINTER(_P)]
            hip.hipGraphInstantiate.argtypes = [C.POINTER(_P), _P, _P, _P, C.c_size_t]
            hip.hipGraphLaunch.argtypes = [_P, _P]
            hip.hipGraphExecDestroy.argtypes = [_P]
            hip.hipGraphDestroy.argtypes = [_P]
            cls._hip = hip
        return cls._hip

    def __init__(self, stream: Stream, fn):
        hip = self._rt()
        self.stream = stream
        self.native = stream.dev.lib.qwhip_stream_native(stream.handle)
        graph, self.exe = _P(), _P()
        if hip.hipStreamBeginCapture(self.native, 1) != 0:          # thread-local capture mode
            raise RuntimeError("hipStreamBeginCapture failed")
        try:
            fn()
        finally:
            rc = hip.hipStreamEndCapture(self.native, C.byref(graph))
        if rc != 0 or not graph.value:
            raise RuntimeError(f"hipStreamEndCapture failed ({rc})")
        rc = hip.hipGraphInstantiate(C.byref(self.exe), graph, None, None, 0)
        hip.hipGraphDestroy(graph)
        if rc != 0:
            raise RuntimeError(f"hipGraphInstantiate failed ({rc})")

    def launch(self) -> None:
        if self._rt().hipGraphLaunch(self.exe, self.native) != 0:
            raise RuntimeError("hipGraphLaunch failed")

    def destroy(self) -> None:
        if self.exe.value:
            self._rt().hipGraphExecDestroy(self.exe)
            self.exe = _P()


class Device:
    def __init__(self, ordinal: int = 0):
        self.lib = load()
        h = _P()
        check(self.lib.qwhip_device_create(ordinal, C.byref(h)))
        self.handle = h.value
        self.stream = Stream(self)

    def caps(self) -> Caps:
        c = Caps()
        check(self.lib.qwhip_device_caps(self.handle, C.byref(c)))
        return c

    def alloc(self, nbytes: int) -> Buffer:
        return Buffer(self, nbytes)

    def put(self, arr: np.ndarray) -> Buffer:
        a = np.ascontiguousarray(arr)
        return Buffer(self, max(a.nbytes, 256)).upload(a)

    def view(self, buf: Buffer, n: int, k: int, kind: int, bits: int = 4, group: int = 32, nbytes: int | None = None,
             offset: int = 0) -> WeightView:
        return WeightView(buf.ptr + offset, buf.nbytes - offset if nbytes is None else nbytes, n, k, kind, bits, group)
