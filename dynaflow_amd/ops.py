"""Torch operators that front the C-ABI kernels (namespace ``dynaflow_hip``).

Each operator is a ``torch.library`` definition with

* a **device implementation** (dispatch key ``CUDA``, which is HIP on ROCm) that
  passes raw device pointers and the current HIP stream to
  ``libdynaflow_hip.so`` through ctypes, and
* a **fake implementation** so the operators can appear inside traced FX graphs
  (dynamo, ``fx.Interpreter`` under fake mode).

There is deliberately no CPU implementation: calling one of these operators on
host tensors, or without the built library, raises.  The operators show up in FX
graphs as ``call_function`` nodes whose ``target.__name__`` starts with the
operator name (``linear``, ``silu_mul``, ...), so ``matching.Op`` patterns such
as ``r"linear(\\.default)?"`` see them like any aten function.

Reference call sites these stand in for: the FX nodes ``linear``, ``silu`` and
``mul`` of the MLP sub-graphs, executed by PyTorch at
dynaflow/runtime/engine.py:381.
"""
from __future__ import annotations

import math
import contextlib
import os
import weakref
import threading

import torch

from dynaflow_amd import _cabi

_lib = torch.library.Library("dynaflow_hip", "DEF")

_lib.define("linear(Tensor x, Tensor weight) -> Tensor")
_lib.define("linear_variant(Tensor x, Tensor weight, int variant) -> Tensor")
_lib.define("silu_mul(Tensor gate, Tensor up, bool round_silu=False) -> Tensor")
_lib.define("gate_up_silu(Tensor x, Tensor w_gate, Tensor w_up) -> Tensor")
_lib.define("rms_norm(Tensor x, Tensor weight, float eps) -> Tensor")
_lib.define("add_rms_norm(Tensor x, Tensor residual, Tensor weight, float eps) -> (Tensor, Tensor)")
_lib.define("transpose_weight(Tensor w) -> Tensor")
_lib.define("rope(Tensor t, Tensor cos, Tensor sin) -> Tensor")
_lib.define("rope_pair(Tensor q, Tensor k, Tensor cos, Tensor sin) -> (Tensor, Tensor)")
_lib.define("causal_attention(Tensor q, Tensor k, Tensor v) -> Tensor")
_lib.define("linear_add(Tensor x, Tensor weight, Tensor residual) -> Tensor")
_lib.define("linear_to_output(Tensor x, Tensor weight) -> Tensor")
_lib.define("linear_multi(Tensor x, Tensor[] weights) -> Tensor[]")
_lib.define("linear_add_to_output(Tensor x, Tensor weight, Tensor residual) -> Tensor")
_lib.define(
    "decode_attention(Tensor qkv, Tensor(a!) k_cache, Tensor(b!) v_cache, Tensor slots, Tensor lengths, "
    "Tensor cos, Tensor sin, int q_heads, int kv_heads) -> Tensor"
)
_lib.define("quant_fp8(Tensor x) -> (Tensor, Tensor)")
_lib.define("silu_mul_quant_fp8(Tensor gate, Tensor up) -> (Tensor, Tensor)")
_lib.define("linear_fp8(Tensor x_q, Tensor w_q, Tensor x_scale, Tensor w_scale) -> Tensor")
_lib.define("linear_fp8_variant(Tensor x_q, Tensor w_q, Tensor x_scale, Tensor w_scale, int variant) -> Tensor")
_lib.define("linear_fp8_to_output(Tensor x_q, Tensor w_q, Tensor x_scale, Tensor w_scale) -> Tensor")
_lib.define(
    "gate_up_silu_quant_fp8(Tensor x_q, Tensor w_gate_q, Tensor w_up_q, Tensor x_scale, Tensor w_gate_scale, "
    "Tensor w_up_scale) -> (Tensor, Tensor)"
)

FP8_DTYPE = torch.float8_e4m3fn
FP8_MAX = 448.0


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _rows(t: torch.Tensor) -> tuple[torch.Tensor, int, int, int]:
    """View ``t[..., D]`` as rows: returns (tensor, M, D, leading dimension).

    A 2-D tensor with unit stride in the last dimension is used as it is (so
    row-strided views such as the halves of a packed gate_up buffer work);
    anything else is flattened, copying only if it has to.
    """
    if t.dim() == 2 and t.stride(1) == 1 and t.stride(0) >= t.shape[1]:
        return t, t.shape[0], t.shape[1], t.stride(0)
    flat = t.reshape(-1, t.shape[-1])
    if flat.stride(1) != 1 or (flat.shape[0] > 1 and flat.stride(0) < flat.shape[1]):
        flat = flat.contiguous()
    ld = flat.stride(0) if flat.shape[0] > 1 else flat.shape[1]
    return flat, flat.shape[0], flat.shape[1], ld


def _require_device(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("dynaflow_hip operators run on the GPU only; got a host tensor")


# ---------------------------------------------------------------- linear
#: split-K workspaces.  Inside a DynaFlow launch: one per (device, engine, nano-batch) - the launches of one
#: nano-batch are chained one after the other whatever streams they run on; different nano-batches, and the
#: forwards of different engines, may overlap and must not share arrival counters.  Outside: one per (device, stream).
_splitk_workspaces: dict[tuple, torch.Tensor] = {}
#: addresses of workspaces that were handed to a launch while its stream was capturing: a graph may replay
#: against them for as long as it lives
_captured_workspaces: set[int] = set()
#: workspaces that were replaced by larger ones and that a captured graph may still point at (one per capture
#: at most: a replaced workspace that no capture ever saw is given back to the allocator)
_retired_workspaces: list[torch.Tensor] = []
#: split K for shapes with too few tiles (DYNAFLOW_SPLIT_K=0 switches it off)
SPLIT_K_ENABLED = os.environ.get("DYNAFLOW_SPLIT_K", "1") != "0"
_launch_options = threading.local()


@contextlib.contextmanager
def launch_options(side_by_side: int = 1):
    """Options for the launches issued inside the block (set by the manager for a forward, from the knobs of its
    configuration).  ``side_by_side=n``: the schedule runs the same sub-graph of ``n`` nano-batches at the same time
    (one stream per nano-batch), so a bf16 GEMM shares the compute units with ``n - 1`` launches of its own shape:
    the kernel plan takes their tiles together - K is split less or not at all, and the tile shape is chosen for
    the rounds that the launches fill together."""
    previous = getattr(_launch_options, "side_by_side", 1)
    _launch_options.side_by_side = max(1, int(side_by_side))
    try:
        yield
    finally:
        _launch_options.side_by_side = previous


def _side_by_side() -> int:
    return getattr(_launch_options, "side_by_side", 1)


def _zeroed_workspace(cache: dict, device: torch.device, stream: int, nbytes: int, clear: int = 65536) -> torch.Tensor:
    """A scratch buffer whose first ``clear`` bytes are zero at first use, kept for the life of the process.

    The kernels that use these buffers (split-K arrival counters) leave them zero, so a buffer made by an
    eager launch (the warm-up that precedes every capture) serves the captured launches of the same
    nano-batch as it is: no allocation and no clearing inside the graph.
    """
    from dynaflow_amd.interface import OperatorHandle
    from dynaflow_amd.runtime.env import peek_op_handle

    handle = peek_op_handle()
    if isinstance(handle, OperatorHandle):
        key = (device.index or 0, "nano-batch", handle._owner, handle.batch_idx)
    else:
        key = (device.index or 0, "stream", stream)
    ws = cache.get(key)
    capturing = torch.cuda.is_current_stream_capturing()
    if ws is not None and ws.numel() >= nbytes:
        if capturing:
            _captured_workspaces.add(ws.data_ptr())
        return ws
    if capturing:
        # No buffer from an eager launch to fall back on: this one comes from the graph's memory pool and its
        # start is zeroed by a fill kernel that is part of the graph (a kernel, not a memset node).
        ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
        rc = _cabi.load().dfhip_fill_u32(ws.data_ptr(), 0, min(nbytes, clear) // 4, stream)
        _cabi.check("dfhip_fill_u32", rc)
        return ws
    if ws is not None:
        if ws.data_ptr() in _captured_workspaces:
            _retired_workspaces.append(ws)
        else:
            ws.record_stream(torch.cuda.current_stream())   # launches already queued on this stream still use it
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=device)
    cache[key] = ws
    return ws


def _splitk_workspace(device: torch.device, stream: int, nbytes: int) -> torch.Tensor:
    return _zeroed_workspace(_splitk_workspaces, device, stream, nbytes)


def _plan_bf16(lib, M: int, N: int, K: int) -> tuple[int, int]:
    """(kernel variant, split of K) for a bf16 GEMM, for as many launches side by side as the forward declared."""
    import ctypes

    variant, split_k = ctypes.c_int(0), ctypes.c_int(1)
    _cabi.check("dfhip_gemm_bf16_plan_shared", lib.dfhip_gemm_bf16_plan_shared(
        M, N, K, _side_by_side(), ctypes.byref(variant), ctypes.byref(split_k)))
    return variant.value, split_k.value


_output_offer = threading.local()


def offer_output_rows(provider) -> None:
    """``provider(rows, cols, dtype, device) -> Tensor [rows, cols] | None`` for the next ``*_to_output`` call."""
    _output_offer.provider = provider


def withdraw_output_rows() -> None:
    _output_offer.provider = None


def _new_output(rows: int, cols: int, dtype: torch.dtype, device: torch.device, to_output: bool) -> torch.Tensor:
    if to_output:
        provider = getattr(_output_offer, "provider", None)
        if provider is not None:
            _output_offer.provider = None
            given = provider(rows, cols, dtype, device)
            if given is not None:
                if tuple(given.shape) != (rows, cols) or given.dtype != dtype or not given.is_contiguous():
                    raise RuntimeError("output rows offered to the operator do not fit its result")
                return given
    return torch.empty((rows, cols), dtype=dtype, device=device)


def _linear_impl(x: torch.Tensor, weight: torch.Tensor, variant: int = -1, split_k_allowed: bool = True,
                 to_output: bool = False) -> torch.Tensor:
    _require_device(x, weight)
    lib = _cabi.load()
    if weight.dim() != 2 or x.shape[-1] != weight.shape[1]:
        raise RuntimeError(f"linear: x[..., {x.shape[-1]}] does not match weight {tuple(weight.shape)}")
    if x.dtype != weight.dtype:
        raise RuntimeError(f"linear: dtype mismatch {x.dtype} vs {weight.dtype}")
    a, M, K, lda = _rows(x)
    w, N, _, ldw = _rows(weight)
    out = _new_output(M, N, x.dtype, x.device, to_output)
    if M > 0:
        if x.dtype == torch.bfloat16:
            if variant == -2:
                split_k_allowed, variant = False, -1
            if variant >= 0:
                rc = lib.dfhip_gemm_bf16_nt_variant(
                    a.data_ptr(), lda, w.data_ptr(), ldw, out.data_ptr(), N, M, N, K, variant, _stream()
                )
                _cabi.check("dfhip_gemm_bf16_nt_variant", rc)
            else:
                planned, split_k = _plan_bf16(lib, M, N, K)
                if split_k > 1 and split_k_allowed and SPLIT_K_ENABLED:
                    stream = _stream()
                    nbytes = lib.dfhip_gemm_bf16_splitk_workspace_bytes(M, N, split_k)
                    ws = _splitk_workspace(x.device, stream, nbytes)
                    rc = lib.dfhip_gemm_bf16_nt_splitk(
                        a.data_ptr(), lda, w.data_ptr(), ldw, out.data_ptr(), N, M, N, K, split_k,
                        ws.data_ptr(), ws.numel(), stream,
                    )
                    _cabi.check("dfhip_gemm_bf16_nt_splitk", rc)
                elif _side_by_side() > 1 and planned != 6:
                    # the plan for launches side by side, not the one the library makes for a lone launch
                    rc = lib.dfhip_gemm_bf16_nt_variant(
                        a.data_ptr(), lda, w.data_ptr(), ldw, out.data_ptr(), N, M, N, K, planned, _stream()
                    )
                    _cabi.check("dfhip_gemm_bf16_nt_variant", rc)
                else:
                    rc = lib.dfhip_gemm_bf16_nt(
                        a.data_ptr(), lda, w.data_ptr(), ldw, out.data_ptr(), N, M, N, K, _stream()
                    )
                    _cabi.check("dfhip_gemm_bf16_nt", rc)
        elif x.dtype == torch.float32:
            rc = lib.dfhip_gemm_f32_nt(
                a.data_ptr(), lda, w.data_ptr(), ldw, out.data_ptr(), N, M, N, K, _stream()
            )
            _cabi.check("dfhip_gemm_f32_nt", rc)
        else:
            raise RuntimeError(f"linear: unsupported dtype {x.dtype}")
    return out.view(*x.shape[:-1], N)


def _linear_fake(x, weight):
    return x.new_empty((*x.shape[:-1], weight.shape[0]))


_lib.impl("linear", lambda x, w: _linear_impl(x, w), "CUDA")
_lib.impl("linear_variant", lambda x, w, v: _linear_impl(x, w, v), "CUDA")
_lib.impl("linear_to_output", lambda x, w: _linear_impl(x, w, to_output=True), "CUDA")
torch.library.register_fake("dynaflow_hip::linear", _linear_fake, lib=_lib)
torch.library.register_fake("dynaflow_hip::linear_to_output", _linear_fake, lib=_lib)
torch.library.register_fake("dynaflow_hip::linear_variant", lambda x, w, v: _linear_fake(x, w), lib=_lib)


# ------------------------------------------- several projections of one activation
class StackedWeightCache:
    """Row-wise concatenations of weight groups (q / k / v, gate / up), one per group of live weights.

    An entry is keyed by what identifies each member as a tensor in memory - device, address, version counter,
    shape and row stride - and it lives exactly as long as its members do: every member carries a finalizer that
    drops the entry, so an address that the allocator hands to a new tensor after a weight was freed never finds
    the old concatenation.  A member written to in place gets a new version counter and with it a new entry
    (the stale one is dropped then); pointing ``w.data`` at another tensor changes the address.  The one update
    no key can see is an in-place write THROUGH ``w.data`` (``w.data.copy_(...)``): callers that update weights
    that way call ``invalidate()`` (``ops.invalidate_stacked_weights``) afterwards, or switch the stacking off
    (``stack_projections=False`` at lowering time, or ``enabled = False`` here).
    """

    def __init__(self) -> None:
        self.enabled = os.environ.get("DYNAFLOW_STACK_WEIGHTS", "1") != "0"
        self._entries: dict[tuple, torch.Tensor] = {}
        self._keys_of_member: dict[int, set] = {}       # id(member) -> keys of the entries it belongs to
        # finalizers run on whatever thread drops the last reference to a weight
        self._lock = threading.RLock()

    @staticmethod
    def key_of(weights) -> tuple:
        return tuple((str(w.device), w.data_ptr(), w._version, tuple(w.shape), w.stride(0)) for w in weights)

    def __len__(self) -> int:
        return len(self._entries)

    def _drop_member(self, member_id: int) -> None:
        with self._lock:
            for key in self._keys_of_member.pop(member_id, ()):
                self._entries.pop(key, None)

    def get(self, weights, build):
        """The concatenation for ``weights``; ``build()`` makes it when there is none (it may return None: no
        entry is kept then)."""
        key = self.key_of(weights)
        with self._lock:
            stacked = self._entries.get(key)
            if stacked is not None:
                return stacked
            stacked = build()
            if stacked is None:
                return None
            for w in weights:
                known = self._keys_of_member.get(id(w))
                if known is None:
                    known = self._keys_of_member[id(w)] = set()
                    weakref.finalize(w, self._drop_member, id(w))
                else:
                    # the same tensor with another address or version: its older concatenations are stale
                    for old in [k for k in known if k != key]:
                        self._entries.pop(old, None)
                        known.discard(old)
                known.add(key)
            self._entries[key] = stacked
            return stacked

    def invalidate(self, weights=None) -> None:
        """Drop every entry (``weights`` None) or the entries that any of ``weights`` belongs to."""
        with self._lock:
            if weights is None:
                self._entries.clear()
                for known in self._keys_of_member.values():
                    known.clear()
                return
            for w in weights:
                for key in list(self._keys_of_member.get(id(w), ())):
                    self._entries.pop(key, None)
                    self._keys_of_member[id(w)].discard(key)


_stacked_weights = StackedWeightCache()


def invalidate_stacked_weights(weights=None) -> None:
    """Forget the stacked copies of weight groups: all of them, or those that any of ``weights`` belongs to.
    To be called after weights were overwritten in place through ``.data`` (the one update the cache cannot see)."""
    _stacked_weights.invalidate(weights)


def _linear_multi_impl(x: torch.Tensor, weights: list[torch.Tensor]) -> list[torch.Tensor]:
    """``[x @ w.T for w in weights]`` as ONE GEMM against the row-wise concatenation of the weights (made on the
    first call and kept); the results are column ranges of one buffer.  q, k and v projections of 4096 + 1024 +
    1024 columns fill the rounds of 256 workgroups as one 6144-column product, not as three."""
    _require_device(x, *weights)
    if x.dtype != torch.bfloat16 or any(w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != x.shape[-1]
                                         or w.shape[0] % 8 for w in weights):
        raise RuntimeError("linear_multi: bf16 activation and [N_i, K] bf16 weights with N_i % 8 == 0 expected")
    def build():
        if torch.cuda.is_current_stream_capturing():
            return None                                        # no allocation that outlives the capture
        return torch.cat([w.detach() for w in weights], dim=0).contiguous()

    stacked = _stacked_weights.get(weights, build) if _stacked_weights.enabled else None
    if stacked is None:
        return [_linear_impl(x, w) for w in weights]
    out = _linear_impl(x, stacked)
    parts, first = [], 0
    for w in weights:
        parts.append(out[..., first:first + w.shape[0]])
        first += w.shape[0]
    return parts


_lib.impl("linear_multi", _linear_multi_impl, "CUDA")
torch.library.register_fake(
    "dynaflow_hip::linear_multi", lambda x, weights: [_linear_fake(x, w) for w in weights], lib=_lib
)


# ------------------------------------------------ projection + residual addition
def _linear_add_impl(x: torch.Tensor, weight: torch.Tensor, residual: torch.Tensor,
                     to_output: bool = False) -> torch.Tensor:
    """``residual + x @ weight.T`` (bf16) in one launch, rounded like the separate linear and add kernels."""
    _require_device(x, weight, residual)
    lib = _cabi.load()
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or residual.dtype != torch.bfloat16:
        raise RuntimeError("linear_add: bf16 tensors expected")
    if weight.dim() != 2 or x.shape[-1] != weight.shape[1]:
        raise RuntimeError(f"linear_add: x[..., {x.shape[-1]}] does not match weight {tuple(weight.shape)}")
    a, M, K, lda = _rows(x)
    w, N, _, ldw = _rows(weight)
    if tuple(residual.shape) != (*x.shape[:-1], N):
        raise RuntimeError(f"linear_add: residual {tuple(residual.shape)} does not match the output")
    r = residual.reshape(M, N)
    if r.stride(1) != 1 or r.stride(0) != N:
        r = r.contiguous()
    out = _new_output(M, N, x.dtype, x.device, to_output)
    if M > 0:
        stream = _stream()
        _, split_k = _plan_bf16(lib, M, N, K)
        ws_ptr, ws_bytes = 0, 0
        if split_k > 1 and SPLIT_K_ENABLED:
            nbytes = lib.dfhip_gemm_bf16_splitk_workspace_bytes(M, N, split_k)
            ws = _splitk_workspace(x.device, stream, nbytes)
            ws_ptr, ws_bytes = ws.data_ptr(), ws.numel()
        else:
            split_k = 1
        rc = lib.dfhip_gemm_bf16_nt_add(
            a.data_ptr(), lda, w.data_ptr(), ldw, r.data_ptr(), out.data_ptr(), N, M, N, K, split_k, ws_ptr,
            ws_bytes, stream,
        )
        _cabi.check("dfhip_gemm_bf16_nt_add", rc)
    return out.view(*x.shape[:-1], N)


_lib.impl("linear_add", _linear_add_impl, "CUDA")
_lib.impl("linear_add_to_output", lambda x, w, r: _linear_add_impl(x, w, r, to_output=True), "CUDA")
torch.library.register_fake("dynaflow_hip::linear_add", lambda x, w, r: _linear_fake(x, w), lib=_lib)
torch.library.register_fake("dynaflow_hip::linear_add_to_output", lambda x, w, r: _linear_fake(x, w), lib=_lib)


# ------------------------------------------- gate/up projection + SiLU*mul epilogue
def _gate_up_silu_impl(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor) -> torch.Tensor:
    """``silu(x @ w_gate.T) * (x @ w_up.T)`` in one launch (bf16, weights in ``linear`` layout)."""
    _require_device(x, w_gate, w_up)
    lib = _cabi.load()
    if x.dtype != torch.bfloat16 or w_gate.dtype != torch.bfloat16 or w_up.dtype != torch.bfloat16:
        raise RuntimeError("gate_up_silu: bf16 only")
    if w_gate.shape != w_up.shape or w_gate.dim() != 2 or x.shape[-1] != w_gate.shape[1]:
        raise RuntimeError("gate_up_silu: shape mismatch")
    a, M, K, lda = _rows(x)
    wg, I, _, ldg = _rows(w_gate)
    wu, _, _, ldu = _rows(w_up)
    if ldg != ldu:
        wg, wu = wg.contiguous(), wu.contiguous()
        ldg = K
    out = torch.empty((M, I), dtype=x.dtype, device=x.device)
    if M > 0:
        rc = lib.dfhip_gemm_bf16_gate_up_silu_shared(
            a.data_ptr(), lda, wg.data_ptr(), wu.data_ptr(), ldg, out.data_ptr(), I, M, I, K, _side_by_side(), _stream()
        )
        _cabi.check("dfhip_gemm_bf16_gate_up_silu", rc)
    return out.view(*x.shape[:-1], I)


_lib.impl("gate_up_silu", _gate_up_silu_impl, "CUDA")
torch.library.register_fake(
    "dynaflow_hip::gate_up_silu", lambda x, wg, wu: x.new_empty((*x.shape[:-1], wg.shape[0])), lib=_lib
)


# -------------------------------------------------------------- silu * mul
def _silu_mul_impl(gate: torch.Tensor, up: torch.Tensor, round_silu: bool = False) -> torch.Tensor:
    _require_device(gate, up)
    lib = _cabi.load()
    if gate.shape != up.shape or gate.dtype != up.dtype:
        raise RuntimeError("silu_mul: gate and up must agree in shape and dtype")
    g, M, D, ldg = _rows(gate)
    u, _, _, ldu = _rows(up)
    out = torch.empty((M, D), dtype=gate.dtype, device=gate.device)
    if M > 0:
        if gate.dtype == torch.bfloat16:
            rc = lib.dfhip_silu_mul_bf16(
                g.data_ptr(), ldg, u.data_ptr(), ldu, out.data_ptr(), D, M, D, int(round_silu), _stream()
            )
            _cabi.check("dfhip_silu_mul_bf16", rc)
        elif gate.dtype == torch.float32:
            rc = lib.dfhip_silu_mul_f32(
                g.data_ptr(), ldg, u.data_ptr(), ldu, out.data_ptr(), D, M, D, _stream()
            )
            _cabi.check("dfhip_silu_mul_f32", rc)
        else:
            raise RuntimeError(f"silu_mul: unsupported dtype {gate.dtype}")
    return out.view(gate.shape)


_lib.impl("silu_mul", _silu_mul_impl, "CUDA")
torch.library.register_fake(
    "dynaflow_hip::silu_mul", lambda gate, up, round_silu=False: torch.empty_like(gate), lib=_lib
)


# ----------------------------------------------------------------- rmsnorm
def _rms_norm_impl(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    _require_device(x, weight)
    lib = _cabi.load()
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise RuntimeError("rms_norm: bf16 only")
    xr = x.reshape(-1, x.shape[-1]).contiguous()
    out = torch.empty_like(xr)
    if xr.shape[0] > 0:
        rc = lib.dfhip_rmsnorm_bf16(
            xr.data_ptr(), None, weight.contiguous().data_ptr(), out.data_ptr(), None,
            xr.shape[0], xr.shape[1], float(eps), _stream(),
        )
        _cabi.check("dfhip_rmsnorm_bf16", rc)
    return out.view(x.shape)


def _add_rms_norm_impl(x, residual, weight, eps):
    _require_device(x, residual, weight)
    lib = _cabi.load()
    if x.dtype != torch.bfloat16 or residual.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise RuntimeError("add_rms_norm: bf16 only")
    xr = x.reshape(-1, x.shape[-1]).contiguous()
    rr = residual.reshape(-1, x.shape[-1]).contiguous()
    out = torch.empty_like(xr)
    res_out = torch.empty_like(xr)
    if xr.shape[0] > 0:
        rc = lib.dfhip_rmsnorm_bf16(
            xr.data_ptr(), rr.data_ptr(), weight.contiguous().data_ptr(), out.data_ptr(),
            res_out.data_ptr(), xr.shape[0], xr.shape[1], float(eps), _stream(),
        )
        _cabi.check("dfhip_rmsnorm_bf16", rc)
    return out.view(x.shape), res_out.view(x.shape)


_lib.impl("rms_norm", _rms_norm_impl, "CUDA")
_lib.impl("add_rms_norm", _add_rms_norm_impl, "CUDA")
torch.library.register_fake("dynaflow_hip::rms_norm", lambda x, w, eps: torch.empty_like(x), lib=_lib)
torch.library.register_fake(
    "dynaflow_hip::add_rms_norm", lambda x, r, w, eps: (torch.empty_like(x), torch.empty_like(x)), lib=_lib
)


def _token_rows(t: torch.Tensor, what: str):
    """[B, S, H, d] with contiguous heads -> (tensor, token stride in elements); a copy only if the tokens
    are not evenly strided rows (a column range of a wider [tokens, columns] buffer is used in place)."""
    if (t.dim() != 4 or t.stride(3) != 1 or t.stride(2) != t.shape[3] or t.stride(1) < t.shape[2] * t.shape[3]
            or t.stride(0) != t.shape[1] * t.stride(1)):
        t = t.contiguous()
    return t, t.stride(1)


# ------------------------------------------------------------------ rope
def _rope_impl(t: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """t [B, S, heads, d] bf16 (contiguous), cos/sin [S, d/2] fp32 -> rotated tensor of the same shape."""
    _require_device(t, cos, sin)
    lib = _cabi.load()
    if t.dtype != torch.bfloat16 or cos.dtype != torch.float32 or sin.dtype != torch.float32 or t.dim() != 4:
        raise RuntimeError("rope: t [B,S,heads,d] bf16 and fp32 tables expected")
    B, S, heads, d = t.shape
    if cos.shape != (S, d // 2) or sin.shape != (S, d // 2):
        raise RuntimeError("rope: table shape mismatch")
    src, ld_src = _token_rows(t, "t")            # a column range of a wider buffer is read in place
    out = torch.empty((B, S, heads, d), dtype=t.dtype, device=t.device)
    if src.numel() > 0:
        rc = lib.dfhip_rope_bf16(
            src.data_ptr(), ld_src, out.data_ptr(), heads * d, cos.contiguous().data_ptr(),
            sin.contiguous().data_ptr(), B * S, heads, d, S, _stream(),
        )
        _cabi.check("dfhip_rope_bf16", rc)
    return out


def _rope_pair_impl(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor):
    """``(rope(q), rope(k))``; when k's heads sit right behind q's in one buffer (column ranges of a stacked
    q / k / v product) both are rotated by ONE launch over all the heads."""
    _require_device(q, k, cos, sin)
    if q.dim() == 4 and k.dim() == 4 and q.dtype == torch.bfloat16 and k.dtype == torch.bfloat16:
        qs, ld_q = _token_rows(q, "q")
        ks, ld_k = _token_rows(k, "k")
        B, S, hq, d = q.shape
        hk = k.shape[2]
        adjacent = (qs is q and ks is k and k.shape[:2] == q.shape[:2] and k.shape[3] == d and ld_q == ld_k
                    and k.data_ptr() == q.data_ptr() + hq * d * q.element_size())
        if adjacent and q.numel() > 0 and cos.shape == (S, d // 2) and sin.shape == (S, d // 2):
            lib = _cabi.load()
            out = torch.empty((B, S, hq + hk, d), dtype=q.dtype, device=q.device)
            rc = lib.dfhip_rope_bf16(
                q.data_ptr(), ld_q, out.data_ptr(), (hq + hk) * d, cos.contiguous().data_ptr(),
                sin.contiguous().data_ptr(), B * S, hq + hk, d, S, _stream(),
            )
            _cabi.check("dfhip_rope_bf16", rc)
            return out[:, :, :hq], out[:, :, hq:]
    return _rope_impl(q, cos, sin), _rope_impl(k, cos, sin)


_lib.impl("rope", _rope_impl, "CUDA")
_lib.impl("rope_pair", _rope_pair_impl, "CUDA")
torch.library.register_fake(
    "dynaflow_hip::rope_pair", lambda q, k, cos, sin: (torch.empty_like(q), torch.empty_like(k)), lib=_lib
)
torch.library.register_fake("dynaflow_hip::rope", lambda t, cos, sin: torch.empty_like(t), lib=_lib)


# ------------------------------------------------------ prefill attention
def _causal_attention_impl(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """q [B, S, Hq, 128], k / v [B, S, Hkv, 128] (bf16) -> softmax(q k^T / sqrt(128), causal) v as [B, S, Hq, 128]."""
    _require_device(q, k, v)
    lib = _cabi.load()
    if q.dtype != torch.bfloat16 or k.dtype != torch.bfloat16 or v.dtype != torch.bfloat16:
        raise RuntimeError("causal_attention: bf16 tensors expected")
    if q.dim() != 4 or k.dim() != 4 or v.shape != k.shape or q.shape[:2] != k.shape[:2] or q.shape[3] != 128 or k.shape[3] != 128:
        raise RuntimeError("causal_attention: q [B,S,Hq,128] and k, v [B,S,Hkv,128] expected")
    B, S, Hq, d = q.shape
    Hkv = k.shape[2]
    if S % 64 != 0 or Hq % Hkv != 0:
        raise RuntimeError("causal_attention: sequence length must be a multiple of 64, q heads a multiple of kv heads")
    q, ld_q = _token_rows(q, "q")
    k, ld_k = _token_rows(k, "k")
    v, ld_v = _token_rows(v, "v")
    out = torch.empty((B, S, Hq, d), dtype=q.dtype, device=q.device)
    if B > 0:
        v_blk = torch.empty((B, Hkv, S // 8, d, 8), dtype=q.dtype, device=q.device)
        stream = _stream()
        rc = lib.dfhip_pack_v_bf16(v.data_ptr(), ld_v, v_blk.data_ptr(), B, S, Hkv, d, stream)
        _cabi.check("dfhip_pack_v_bf16", rc)
        rc = lib.dfhip_causal_attention_bf16(
            q.data_ptr(), ld_q, k.data_ptr(), ld_k, v_blk.data_ptr(), out.data_ptr(), Hq * d, B, S, Hq, Hkv, d,
            1.0 / math.sqrt(d), stream,
        )
        _cabi.check("dfhip_causal_attention_bf16", rc)
    return out


_lib.impl("causal_attention", _causal_attention_impl, "CUDA")
torch.library.register_fake("dynaflow_hip::causal_attention", lambda q, k, v: torch.empty_like(q), lib=_lib)


# ------------------------------------------------------- decode attention
def _decode_attention_impl(qkv, k_cache, v_cache, slots, lengths, cos, sin, q_heads: int, kv_heads: int):
    """RoPE + cache append + attention of one new token per sequence (see ``dynaflow_amd.decode``).

    qkv [T, (q_heads + 2 kv_heads) * 128] bf16; k_cache [slots, kv_heads, capacity, 128];
    v_cache [slots, kv_heads, capacity / 8, 128, 8]; slots, lengths [T] int32; cos, sin [rows, 64] fp32.
    """
    _require_device(qkv, k_cache, v_cache, slots, lengths, cos, sin)
    lib = _cabi.load()
    d = 128
    if qkv.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16:
        raise RuntimeError("decode_attention: bf16 tensors expected")
    if slots.dtype != torch.int32 or lengths.dtype != torch.int32 or cos.dtype != torch.float32 or sin.dtype != torch.float32:
        raise RuntimeError("decode_attention: int32 slots / lengths and fp32 tables expected")
    if k_cache.dim() != 4 or v_cache.dim() != 5 or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise RuntimeError("decode_attention: contiguous k_cache [S,H,C,128] and v_cache [S,H,C/8,128,8] expected")
    num_slots, kvh, capacity, hd = k_cache.shape
    if hd != d or kvh != kv_heads or tuple(v_cache.shape) != (num_slots, kvh, capacity // 8, d, 8):
        raise RuntimeError("decode_attention: cache shapes do not match")
    if qkv.dim() != 2 or qkv.shape[1] != (q_heads + 2 * kv_heads) * d or qkv.stride(1) != 1:
        raise RuntimeError("decode_attention: qkv [T, (q_heads + 2 kv_heads) * 128] expected")
    T = qkv.shape[0]
    if slots.shape != (T,) or lengths.shape != (T,) or cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != d // 2:
        raise RuntimeError("decode_attention: slots / lengths / table shapes do not match")
    slots, lengths, cos, sin = slots.contiguous(), lengths.contiguous(), cos.contiguous(), sin.contiguous()
    out = torch.empty((T, q_heads * d), dtype=qkv.dtype, device=qkv.device)
    if T > 0:
        # rotation, cache append and attention in one launch
        rc = lib.dfhip_decode_attention_append_bf16(
            qkv.data_ptr(), qkv.stride(0), k_cache.data_ptr(), v_cache.data_ptr(), slots.data_ptr(),
            lengths.data_ptr(), cos.data_ptr(), sin.data_ptr(), out.data_ptr(), q_heads * d, T, q_heads, kv_heads, d,
            num_slots, capacity, cos.shape[0], 1.0 / math.sqrt(d), _stream(),
        )
        _cabi.check("dfhip_decode_attention_append_bf16", rc)
    return out


_lib.impl("decode_attention", _decode_attention_impl, "CUDA")
torch.library.register_fake(
    "dynaflow_hip::decode_attention",
    lambda qkv, k_cache, v_cache, slots, lengths, cos, sin, q_heads, kv_heads: qkv.new_empty(
        (qkv.shape[0], q_heads * 128)
    ),
    lib=_lib,
)


# ------------------------------------------------------ weight re-layout
def _transpose_weight_impl(w: torch.Tensor) -> torch.Tensor:
    """[K, N] (``x @ W`` convention) -> [N, K] (``linear`` convention), bf16."""
    _require_device(w)
    lib = _cabi.load()
    if w.dim() != 2 or w.dtype != torch.bfloat16:
        raise RuntimeError("transpose_weight: 2-D bf16 only")
    src, K, N, ld = _rows(w)
    out = torch.empty((N, K), dtype=w.dtype, device=w.device)
    rc = lib.dfhip_transpose_bf16(src.data_ptr(), ld, out.data_ptr(), K, K, N, _stream())
    _cabi.check("dfhip_transpose_bf16", rc)
    return out


_lib.impl("transpose_weight", _transpose_weight_impl, "CUDA")
torch.library.register_fake(
    "dynaflow_hip::transpose_weight", lambda w: w.new_empty((w.shape[1], w.shape[0])), lib=_lib
)


# --------------------------------------------------------------------- fp8
def _fill_zero(t: torch.Tensor) -> None:
    rc = _cabi.load().dfhip_fill_u32(t.data_ptr(), 0, t.numel(), _stream())
    _cabi.check("dfhip_fill_u32", rc)


def _quant_fp8_impl(x: torch.Tensor):
    """Per-tensor dynamic quantisation: returns (e4m3fn tensor, scale[1] fp32)."""
    _require_device(x)
    lib = _cabi.load()
    if x.dtype != torch.bfloat16:
        raise RuntimeError("quant_fp8: bf16 input only")
    xr, M, D, ld = _rows(x)
    amax = torch.empty(1, dtype=torch.float32, device=x.device)
    scale = torch.empty(1, dtype=torch.float32, device=x.device)
    q = torch.empty((M, D), dtype=FP8_DTYPE, device=x.device)
    _fill_zero(amax)
    rc = lib.dfhip_absmax_bf16(xr.data_ptr(), ld, M, D, amax.data_ptr(), _stream())
    _cabi.check("dfhip_absmax_bf16", rc)
    rc = lib.dfhip_quant_fp8_bf16(
        xr.data_ptr(), ld, q.data_ptr(), D, M, D, amax.data_ptr(), scale.data_ptr(), _stream()
    )
    _cabi.check("dfhip_quant_fp8_bf16", rc)
    return q.view(x.shape), scale


def _silu_mul_quant_fp8_impl(gate: torch.Tensor, up: torch.Tensor):
    """silu(gate)*up, re-quantised per tensor: returns (e4m3fn tensor, scale[1])."""
    _require_device(gate, up)
    lib = _cabi.load()
    if gate.dtype != torch.bfloat16 or gate.shape != up.shape or up.dtype != torch.bfloat16:
        raise RuntimeError("silu_mul_quant_fp8: two bf16 tensors of one shape")
    g, M, D, ldg = _rows(gate)
    u, _, _, ldu = _rows(up)
    act = torch.empty((M, D), dtype=torch.bfloat16, device=gate.device)
    amax = torch.empty(1, dtype=torch.float32, device=gate.device)
    scale = torch.empty(1, dtype=torch.float32, device=gate.device)
    q = torch.empty((M, D), dtype=FP8_DTYPE, device=gate.device)
    _fill_zero(amax)
    rc = lib.dfhip_silu_mul_absmax_bf16(
        g.data_ptr(), ldg, u.data_ptr(), ldu, act.data_ptr(), D, M, D, amax.data_ptr(), _stream()
    )
    _cabi.check("dfhip_silu_mul_absmax_bf16", rc)
    rc = lib.dfhip_quant_fp8_bf16(
        act.data_ptr(), D, q.data_ptr(), D, M, D, amax.data_ptr(), scale.data_ptr(), _stream()
    )
    _cabi.check("dfhip_quant_fp8_bf16", rc)
    return q.view(gate.shape), scale


def _gate_up_silu_quant_fp8_impl(x_q, w_gate_q, w_up_q, x_scale, w_gate_scale, w_up_scale):
    """The fp8 gate and up projections with SiLU*mul as the GEMM's epilogue, then the re-quantisation:
    returns what ``silu_mul_quant_fp8(linear_fp8(x, w_gate), linear_fp8(x, w_up))`` returns, bit for bit."""
    _require_device(x_q, w_gate_q, w_up_q, x_scale, w_gate_scale, w_up_scale)
    lib = _cabi.load()
    if x_q.dtype != FP8_DTYPE or w_gate_q.dtype != FP8_DTYPE or w_up_q.dtype != FP8_DTYPE:
        raise RuntimeError("gate_up_silu_quant_fp8: e4m3fn operands only")
    if any(t.dtype != torch.float32 for t in (x_scale, w_gate_scale, w_up_scale)):
        raise RuntimeError("gate_up_silu_quant_fp8: fp32 scales only")
    a, M, K, lda = _rows(x_q)
    wg, I, Kw, ldg = _rows(w_gate_q)
    wu, Iu, Ku, ldu = _rows(w_up_q)
    if K != Kw or K != Ku or I != Iu or w_gate_scale.numel() != I or w_up_scale.numel() != I or x_scale.numel() != 1:
        raise RuntimeError("gate_up_silu_quant_fp8: shape mismatch")
    if ldg != ldu:
        wg, wu = wg.contiguous(), wu.contiguous()
        ldg = K
    act = torch.empty((M, I), dtype=torch.bfloat16, device=x_q.device)
    amax = torch.empty(1, dtype=torch.float32, device=x_q.device)
    scale = torch.empty(1, dtype=torch.float32, device=x_q.device)
    q = torch.empty((M, I), dtype=FP8_DTYPE, device=x_q.device)
    if M > 0:
        _fill_zero(amax)
        rc = lib.dfhip_gemm_fp8_gate_up_silu_absmax(
            a.data_ptr(), lda, wg.data_ptr(), wu.data_ptr(), ldg, act.data_ptr(), I, x_scale.data_ptr(),
            w_gate_scale.contiguous().data_ptr(), w_up_scale.contiguous().data_ptr(), amax.data_ptr(), M, I, K,
            _stream(),
        )
        _cabi.check("dfhip_gemm_fp8_gate_up_silu_absmax", rc)
        rc = lib.dfhip_quant_fp8_bf16(act.data_ptr(), I, q.data_ptr(), I, M, I, amax.data_ptr(), scale.data_ptr(),
                                      _stream())
        _cabi.check("dfhip_quant_fp8_bf16", rc)
    return q.view(*x_q.shape[:-1], I), scale


def _linear_fp8_impl(x_q, w_q, x_scale, w_scale, variant: int = -1, to_output: bool = False):
    _require_device(x_q, w_q, x_scale, w_scale)
    lib = _cabi.load()
    if x_q.dtype != FP8_DTYPE or w_q.dtype != FP8_DTYPE:
        raise RuntimeError("linear_fp8: e4m3fn operands only")
    if x_scale.dtype != torch.float32 or w_scale.dtype != torch.float32:
        raise RuntimeError("linear_fp8: fp32 scales only")
    a, M, K, lda = _rows(x_q)
    w, N, Kw, ldw = _rows(w_q)
    if K != Kw or w_scale.numel() != N or x_scale.numel() != 1:
        raise RuntimeError("linear_fp8: shape mismatch")
    out = _new_output(M, N, torch.bfloat16, x_q.device, to_output)
    if M > 0:
        rc = lib.dfhip_gemm_fp8_nt_variant(
            a.data_ptr(), lda, w.data_ptr(), ldw, out.data_ptr(), N,
            x_scale.data_ptr(), w_scale.contiguous().data_ptr(), M, N, K, variant, _stream(),
        )
        _cabi.check("dfhip_gemm_fp8_nt_variant", rc)
    return out.view(*x_q.shape[:-1], N)


_lib.impl("quant_fp8", _quant_fp8_impl, "CUDA")
_lib.impl("silu_mul_quant_fp8", _silu_mul_quant_fp8_impl, "CUDA")
_lib.impl("gate_up_silu_quant_fp8", _gate_up_silu_quant_fp8_impl, "CUDA")
torch.library.register_fake(
    "dynaflow_hip::gate_up_silu_quant_fp8",
    lambda x_q, wg, wu, xs, wgs, wus: (x_q.new_empty((*x_q.shape[:-1], wg.shape[0]), dtype=FP8_DTYPE),
                                       x_q.new_empty((1,), dtype=torch.float32)),
    lib=_lib,
)
_lib.impl("linear_fp8", lambda x_q, w_q, xs, ws: _linear_fp8_impl(x_q, w_q, xs, ws), "CUDA")
_lib.impl("linear_fp8_variant", lambda x_q, w_q, xs, ws, v: _linear_fp8_impl(x_q, w_q, xs, ws, v), "CUDA")
_lib.impl("linear_fp8_to_output", lambda x_q, w_q, xs, ws: _linear_fp8_impl(x_q, w_q, xs, ws, to_output=True), "CUDA")
torch.library.register_fake(
    "dynaflow_hip::quant_fp8",
    lambda x: (x.new_empty(x.shape, dtype=FP8_DTYPE), x.new_empty((1,), dtype=torch.float32)),
    lib=_lib,
)
torch.library.register_fake(
    "dynaflow_hip::silu_mul_quant_fp8",
    lambda g, u: (g.new_empty(g.shape, dtype=FP8_DTYPE), g.new_empty((1,), dtype=torch.float32)),
    lib=_lib,
)
torch.library.register_fake(
    "dynaflow_hip::linear_fp8",
    lambda x_q, w_q, xs, ws: x_q.new_empty((*x_q.shape[:-1], w_q.shape[0]), dtype=torch.bfloat16),
    lib=_lib,
)
torch.library.register_fake(
    "dynaflow_hip::linear_fp8_to_output",
    lambda x_q, w_q, xs, ws: x_q.new_empty((*x_q.shape[:-1], w_q.shape[0]), dtype=torch.bfloat16),
    lib=_lib,
)
torch.library.register_fake(
    "dynaflow_hip::linear_fp8_variant",
    lambda x_q, w_q, xs, ws, v: x_q.new_empty((*x_q.shape[:-1], w_q.shape[0]), dtype=torch.bfloat16),
    lib=_lib,
)

linear = torch.ops.dynaflow_hip.linear
linear_variant = torch.ops.dynaflow_hip.linear_variant
silu_mul = torch.ops.dynaflow_hip.silu_mul
gate_up_silu = torch.ops.dynaflow_hip.gate_up_silu
rms_norm = torch.ops.dynaflow_hip.rms_norm
add_rms_norm = torch.ops.dynaflow_hip.add_rms_norm
transpose_weight = torch.ops.dynaflow_hip.transpose_weight
rope = torch.ops.dynaflow_hip.rope
rope_pair = torch.ops.dynaflow_hip.rope_pair
decode_attention = torch.ops.dynaflow_hip.decode_attention
causal_attention = torch.ops.dynaflow_hip.causal_attention
linear_add = torch.ops.dynaflow_hip.linear_add
linear_to_output = torch.ops.dynaflow_hip.linear_to_output
linear_multi = torch.ops.dynaflow_hip.linear_multi
linear_add_to_output = torch.ops.dynaflow_hip.linear_add_to_output
quant_fp8 = torch.ops.dynaflow_hip.quant_fp8
silu_mul_quant_fp8 = torch.ops.dynaflow_hip.silu_mul_quant_fp8
linear_fp8 = torch.ops.dynaflow_hip.linear_fp8
linear_fp8_variant = torch.ops.dynaflow_hip.linear_fp8_variant
linear_fp8_to_output = torch.ops.dynaflow_hip.linear_fp8_to_output
gate_up_silu_quant_fp8 = torch.ops.dynaflow_hip.gate_up_silu_quant_fp8
