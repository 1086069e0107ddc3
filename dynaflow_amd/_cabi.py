"""ctypes binding of ``libdynaflow_hip.so`` (the C ABI in include/dynaflow_hip.h).

Loading is explicit and loud: there is no substitute implementation.  If the
shared library has not been built, ``load()`` raises ``KernelLibraryMissing``
naming the build command, and every operator that needs a kernel propagates
that error.

The reference has no kernel FFI on this path (its sub-graphs call PyTorch,
dynaflow/runtime/engine.py:381); the callables built on this binding go where
it keeps a sub-graph's callable (dynaflow/executor/compiler.py:69-85).
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_uint32, c_void_p

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libdynaflow_hip.so"
LIB_PATH = os.path.join(_PKG_DIR, LIB_NAME)


class KernelLibraryMissing(RuntimeError):
    pass


class KernelError(RuntimeError):
    """A C-ABI call returned a negative status."""

    def __init__(self, entry: str, status: int, text: str) -> None:
        super().__init__(f"{entry} failed: {text} (status {status})")
        self.entry = entry
        self.status = status


class DeviceInfo(ctypes.Structure):
    _fields_ = [
        ("compute_units", c_int),
        ("clock_khz", c_int),
        ("memory_clock_khz", c_int),
        ("memory_bus_bits", c_int),
        ("lds_bytes_per_block", c_int),
        ("wavefront_size", c_int),
        ("arch_name", ctypes.c_char * 64),
    ]


_P = c_void_p
_F = ctypes.POINTER(c_float)

#: name -> (restype, argtypes); the complete export list of include/dynaflow_hip.h
SIGNATURES: dict[str, tuple] = {
    "dfhip_version": (c_int, []),
    "dfhip_arch": (c_char_p, []),
    "dfhip_status_string": (c_char_p, [c_int]),
    "dfhip_device_info_get": (c_int, [c_int, ctypes.POINTER(DeviceInfo)]),
    "dfhip_gemm_bf16_nt": (c_int, [_P, c_int64, _P, c_int64, _P, c_int64, c_int, c_int, c_int, _P]),
    "dfhip_gemm_bf16_nt_variant": (
        c_int,
        [_P, c_int64, _P, c_int64, _P, c_int64, c_int, c_int, c_int, c_int, _P],
    ),
    "dfhip_gemm_bf16_plan": (c_int, [c_int, c_int, c_int, ctypes.POINTER(c_int), ctypes.POINTER(c_int)]),
    "dfhip_gemm_bf16_plan_shared": (c_int, [c_int, c_int, c_int, c_int, ctypes.POINTER(c_int), ctypes.POINTER(c_int)]),
    "dfhip_gemm_bf16_splitk_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "dfhip_gemm_bf16_nt_splitk": (
        c_int,
        [_P, c_int64, _P, c_int64, _P, c_int64, c_int, c_int, c_int, c_int, _P, c_size_t, _P],
    ),
    "dfhip_gemm_bf16_splitk_work": (c_int, [c_int, c_int, c_int, ctypes.POINTER(c_int), ctypes.POINTER(c_int)]),
    "dfhip_gemm_bf16_nt_splitk_static": (
        c_int,
        [_P, c_int64, _P, c_int64, _P, c_int64, c_int, c_int, c_int, c_int, _P],
    ),
    "dfhip_gemm_bf16_nt_add": (c_int, [_P, c_int64, _P, c_int64, _P, _P, c_int64, c_int, c_int, c_int, c_int, _P,
                                       c_size_t, _P]),
    "dfhip_gemm_bf16_gate_up_silu": (c_int, [_P, c_int64, _P, _P, c_int64, _P, c_int64, c_int, c_int, c_int, _P]),
    "dfhip_gemm_bf16_gate_up_silu_shared": (c_int, [_P, c_int64, _P, _P, c_int64, _P, c_int64, c_int, c_int, c_int,
                                                    c_int, _P]),
    "dfhip_gemm_f32_nt": (c_int, [_P, c_int64, _P, c_int64, _P, c_int64, c_int, c_int, c_int, _P]),
    "dfhip_gemm_fp8_nt": (
        c_int,
        [_P, c_int64, _P, c_int64, _P, c_int64, _P, _P, c_int, c_int, c_int, _P],
    ),
    "dfhip_gemm_fp8_nt_variant": (
        c_int,
        [_P, c_int64, _P, c_int64, _P, c_int64, _P, _P, c_int, c_int, c_int, c_int, _P],
    ),
    "dfhip_gemm_fp8_gate_up_silu_absmax": (c_int, [_P, c_int64, _P, _P, c_int64, _P, c_int64, _P, _P, _P, _P, c_int,
                                                     c_int, c_int, _P]),
    "dfhip_silu_mul_bf16": (c_int, [_P, c_int64, _P, c_int64, _P, c_int64, c_int, c_int, c_int, _P]),
    "dfhip_silu_mul_f32": (c_int, [_P, c_int64, _P, c_int64, _P, c_int64, c_int, c_int, _P]),
    "dfhip_rmsnorm_bf16": (c_int, [_P, _P, _P, _P, _P, c_int, c_int, c_float, _P]),
    "dfhip_rope_bf16": (c_int, [_P, c_int64, _P, c_int64, _P, _P, c_int, c_int, c_int, c_int, _P]),
    "dfhip_pack_v_bf16": (c_int, [_P, c_int64, _P, c_int, c_int, c_int, c_int, _P]),
    "dfhip_causal_attention_bf16": (c_int, [_P, c_int64, _P, c_int64, _P, _P, c_int64, c_int, c_int, c_int, c_int,
                                            c_int, c_float, _P]),
    "dfhip_rope_kv_append_bf16": (c_int, [_P, c_int64, _P, c_int64, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int,
                                          c_int, c_int, c_int, _P]),
    "dfhip_decode_attention_bf16": (c_int, [_P, c_int64, _P, _P, _P, _P, _P, c_int64, c_int, c_int, c_int, c_int,
                                            c_int, c_int, ctypes.c_float, _P]),
    "dfhip_decode_attention_append_bf16": (c_int, [_P, c_int64, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int, c_int,
                                                   c_int, c_int, c_int, c_int, c_int, ctypes.c_float, _P]),
    "dfhip_transpose_bf16": (c_int, [_P, c_int64, _P, c_int64, c_int, c_int, _P]),
    "dfhip_absmax_bf16": (c_int, [_P, c_int64, c_int, c_int, _P, _P]),
    "dfhip_quant_fp8_bf16": (c_int, [_P, c_int64, _P, c_int64, c_int, c_int, _P, _P, _P]),
    "dfhip_silu_mul_absmax_bf16": (
        c_int,
        [_P, c_int64, _P, c_int64, _P, c_int64, c_int, c_int, _P, _P],
    ),
    "dfhip_fill_u32": (c_int, [_P, c_uint32, c_int64, _P]),
}

_lib: ctypes.CDLL | None = None


def is_built() -> bool:
    return os.path.exists(LIB_PATH)


def load() -> ctypes.CDLL:
    """Load the library once and attach the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not is_built():
        raise KernelLibraryMissing(
            f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_PKG_DIR, 'csrc')}` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'` from the repository root)"
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = header and library disagree
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(entry: str, status: int) -> None:
    """Turn a negative status into ``KernelError``."""
    if status != 0:
        text = load().dfhip_status_string(status).decode()
        raise KernelError(entry, status, text)


def device_info(device: int = 0) -> dict:
    info = DeviceInfo()
    check("dfhip_device_info_get", load().dfhip_device_info_get(device, ctypes.byref(info)))
    return {
        "compute_units": info.compute_units,
        "clock_khz": info.clock_khz,
        "memory_clock_khz": info.memory_clock_khz,
        "memory_bus_bits": info.memory_bus_bits,
        "lds_bytes_per_block": info.lds_bytes_per_block,
        "wavefront_size": info.wavefront_size,
        "arch_name": info.arch_name.decode(),
    }
