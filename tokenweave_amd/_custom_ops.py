"""Op shims with the reference's names and argument lists.

Mirror of ``vllm/_custom_ops.py:176-221``: every function mutates its tensor
arguments in place and returns ``None``.  The same schema strings the reference
registers in ``csrc/torch_bindings.cpp:133-171`` are registered here under the
``tokenweave_amd`` namespace, so ``torch.ops.tokenweave_amd.fused_add_rms_norm``
is callable exactly like ``torch.ops._C.fused_add_rms_norm``.

Each op validates on the host what the HIP kernel assumes (device, dtype, row
contiguity, shapes) and then enqueues one kernel on the current torch stream of
the tensor's device through the C ABI.  There is no CPU implementation: calling
an op with CPU tensors, or without the built library, raises.
"""
from __future__ import annotations

import bisect
import ctypes
import itertools
import os
import types
import threading
import warnings
import weakref
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import _lib

_DTYPE_CODE = {torch.bfloat16: _lib.TW_DTYPE_BF16, torch.float16: _lib.TW_DTYPE_F16,
               torch.float32: _lib.TW_DTYPE_F32}

# The ops registered with torch's dispatcher by the compiled binding
# (csrc/tw_torch_binding.cpp -> libtokenweave_amd_torch.so, TORCH_LIBRARY with the
# reference's schema strings).  When it has been built the public functions of this
# module are one call into it, as vllm/_custom_ops.py is one call into torch.ops._C;
# without it the same schemas are registered from Python further down and every op
# goes through ctypes (`via_ctypes` always names that route).
BINDING_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libtokenweave_amd_torch.so")
COMPILED_BINDING = False
if os.path.exists(BINDING_PATH) and os.environ.get("TOKENWEAVE_AMD_NO_COMPILED_BINDING") != "1":
    try:
        torch.ops.load_library(BINDING_PATH)
        COMPILED_BINDING = True
    except OSError as e:   # e.g. built against another torch: the ctypes route serves every op
        warnings.warn(f"{BINDING_PATH} could not be loaded ({e}); tokenweave_amd registers its ops "
                      "from Python and calls the HIP library through ctypes instead", RuntimeWarning)
_T = torch.ops.tokenweave_amd

# Message of the reference's launchers (csrc/tokenweave_fused_kernels.cu:259).
ALIGNMENT_MESSAGE = ("Input, residual, and weight tensors must be 16-byte aligned and "
                     "hidden_size must be divisible by 8 for optimized kernel.")


# ---------------------------------------------------------------------------
# host-side checks
# ---------------------------------------------------------------------------
def _rows(t: torch.Tensor) -> Tuple[int, int]:
    """(num_tokens, hidden_size) as the reference computes them
    (csrc/layernorm_kernels.cu:198-199)."""
    if t.dim() < 1:
        raise RuntimeError("expected a tensor with at least one dimension")
    hidden = t.size(-1)
    return (t.numel() // hidden if hidden else 0), hidden


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _check_tensor(name: str, t: torch.Tensor, dtype: torch.dtype, device: torch.device) -> None:
    # one pass for the common case; the individual checks below only word the error
    if (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == dtype and t.device == device
            and t.is_contiguous()):
        return
    _require(isinstance(t, torch.Tensor), f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise RuntimeError(
            f"{name} is on {t.device}: tokenweave_amd ops run on the GPU only "
            "(there is no CPU implementation)")
    _require(t.device == device, f"{name} is on {t.device}, expected {device}")
    if t.dtype != dtype:
        raise RuntimeError(f"{name} has dtype {t.dtype}, expected {dtype}")
    _require(t.is_contiguous(),
             f"{name} must be row-contiguous (stride(-1) == 1, stride(-2) == hidden_size); "
             f"got shape {tuple(t.shape)} stride {tuple(t.stride())}")


def _check_weight(weight: torch.Tensor, hidden: int, dtype, device) -> None:
    _check_tensor("weight", weight, dtype, device)
    if weight.numel() != hidden:
        raise RuntimeError(f"weight has {weight.numel()} elements, expected hidden_size {hidden}")


def _dtype_code(name: str, t: torch.Tensor) -> int:
    code = _DTYPE_CODE.get(t.dtype)
    if code is None:
        # AT_DISPATCH_SWITCH wording (csrc/dispatch_utils.h:14-21)
        raise NotImplementedError(f'"{name}" not implemented for \'{t.dtype}\'')
    return code


def _require_bf16(name: str, t: torch.Tensor) -> None:
    if t.dtype != torch.bfloat16:
        # csrc/dispatch_utils.h:23-27: the TokenWeave kernels dispatch bf16 only
        raise NotImplementedError(f'"{name}" not implemented for \'{t.dtype}\'')


# torch's raw accessors (what its own compiled-kernel launchers use) skip the Stream /
# device object construction of the public calls; fall back to those if they are gone.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream_ptr(t: torch.Tensor) -> int:
    """hipStream_t of the current stream of the tensor's device, as an integer."""
    if _raw_stream is not None:
        idx = t.device.index
        return _raw_stream(idx if idx is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(t.device).cuda_stream


class _DeviceGuard:
    """Make the tensor's device current for the duration of the launch
    (OptionalCUDAGuard in the reference, csrc/tokenweave_fused_kernels.cu:239).
    The usual case — it already is — costs one integer comparison."""
    __slots__ = ("guard",)

    def __init__(self):
        self.guard = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        if self.guard is not None:
            self.guard.__exit__(*exc)
            self.guard = None


_NO_SWITCH = _DeviceGuard()


def _on_device(t: torch.Tensor):
    idx = t.device.index
    cur = _raw_device() if _raw_device is not None else torch.cuda.current_device()
    if idx is None or idx == cur:
        return _NO_SWITCH
    g = _DeviceGuard()
    g.guard = torch.cuda.device(idx)
    g.guard.__enter__()
    return g


def _cap(max_ctas: Optional[int]) -> int:
    return 0 if max_ctas is None else int(max_ctas)


# ---------------------------------------------------------------------------
# layer norm ops (vllm/_custom_ops.py:176-182)
# ---------------------------------------------------------------------------
def rms_norm(out: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
             epsilon: float) -> None:
    code = _dtype_code("rms_norm_kernel", input)
    _check_tensor("input", input, input.dtype, input.device)
    _check_tensor("out", out, input.dtype, input.device)
    T, H = _rows(input)
    _require(out.shape == input.shape, "out and input must have the same shape")
    _check_weight(weight, H, input.dtype, input.device)
    with _on_device(input):
        _lib.check(_lib.lib().tw_rms_norm(out.data_ptr(), input.data_ptr(), weight.data_ptr(),
                                          T, H, epsilon, code, _stream_ptr(input)))


def fused_add_rms_norm(input: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                       epsilon: float) -> None:
    code = _dtype_code("fused_add_rms_norm_kernel", input)
    _check_tensor("input", input, input.dtype, input.device)
    _check_tensor("residual", residual, input.dtype, input.device)
    T, H = _rows(input)
    _require(residual.shape == input.shape, "input and residual must have the same shape")
    _check_weight(weight, H, input.dtype, input.device)
    with _on_device(input):
        _lib.check(_lib.lib().tw_fused_add_rms_norm(
            input.data_ptr(), residual.data_ptr(), weight.data_ptr(), T, H, epsilon, code,
            _stream_ptr(input)))


# ---------------------------------------------------------------------------
# TokenWeave ops (vllm/_custom_ops.py:184-207)
# ---------------------------------------------------------------------------
def rms_norm_inplace(out: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
                     epsilon: float) -> None:
    code = _dtype_code("rms_norm_inplace_kernel", input)
    _check_tensor("input", input, input.dtype, input.device)
    _check_tensor("out", out, input.dtype, input.device)
    T, H = _rows(input)
    _require(out.shape == input.shape, "out and input must have the same shape")
    _check_weight(weight, H, input.dtype, input.device)
    with _on_device(input):
        _lib.check(_lib.lib().tw_rms_norm_inplace(
            out.data_ptr(), input.data_ptr(), weight.data_ptr(), T, H, epsilon, code,
            _stream_ptr(input)))


def fused_add_rms_norm_cta(input: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                           MAX_CTAS: int, epsilon: float) -> None:
    _require_bf16("fused_add_rms_norm_cta_kernel", input)
    _check_tensor("input", input, torch.bfloat16, input.device)
    _check_tensor("residual", residual, torch.bfloat16, input.device)
    T, H = _rows(input)
    _require(residual.shape == input.shape, "input and residual must have the same shape")
    _check_weight(weight, H, torch.bfloat16, input.device)
    with _on_device(input):
        _lib.check(_lib.lib().tw_fused_add_rms_norm_cta(
            input.data_ptr(), residual.data_ptr(), weight.data_ptr(), T, H, _cap(MAX_CTAS),
            epsilon, _stream_ptr(input)))


# --- one-GPU stand-in for the symmetric-memory address space -----------------
# The reference passes `mcptr`, one multicast address that names the same offset
# in every rank's staging buffer (layernorm.py:79).  On one GPU the P staging
# buffers are slots of one allocation; a registered region tells the shim the
# distance between slots so that `mcptr + p * stride` is partial p.
# Regions are kept sorted by base address (bisect) behind a lock; the region that served
# the last call is tried first, so the usual lookup is a few comparisons.
_REGIONS: List[Tuple[int, int, int, int, "weakref.ref"]] = []  # (base, stride, slots, usable, owner)
_REGION_BASES: List[int] = []
_REGIONS_LOCK = threading.Lock()
_REGION_TOKENS = itertools.count(1)
_LAST_REGION: Optional[Tuple[int, int, int, int, "weakref.ref"]] = None


def register_partials_region(base_ptr: int, stride_bytes: int, slots: int, owner,
                             usable_bytes: Optional[int] = None) -> None:
    """Declare [base_ptr, base_ptr + slots*stride_bytes) as `slots` equally spaced
    partial-sum buffers of `usable_bytes` each (default: the whole stride).  `owner` is
    weakly referenced; the region is dropped with it."""
    global _LAST_REGION
    _require(stride_bytes > 0 and stride_bytes % 16 == 0, "slot stride must be a positive multiple of 16")
    _require(1 <= slots <= _lib.TW_MAX_PARTIALS, f"slots must be in [1, {_lib.TW_MAX_PARTIALS}]")
    usable = int(stride_bytes if usable_bytes is None else usable_bytes)
    _require(0 < usable <= stride_bytes, "usable bytes of a slot must fit its stride")
    entry = (int(base_ptr), int(stride_bytes), int(slots), usable, weakref.ref(owner))
    if COMPILED_BINDING:
        # the compiled ops keep their own table; the entry goes when the owner does
        token = next(_REGION_TOKENS)
        _T.register_partials_region(entry[0], entry[1], entry[2], usable, token)
        weakref.finalize(owner, _T.unregister_partials_region, entry[0], token)
    with _REGIONS_LOCK:
        live = [r for r in _REGIONS if r[4]() is not None and r[0] != entry[0]]
        live.append(entry)
        live.sort(key=lambda r: r[0])
        _REGIONS[:] = live
        _REGION_BASES[:] = [r[0] for r in live]
        _LAST_REGION = None


def _find_region(mcptr: int):
    global _LAST_REGION
    r = _LAST_REGION
    if r is not None and r[0] <= mcptr < r[0] + r[1] and r[4]() is not None:
        return r
    with _REGIONS_LOCK:
        i = bisect.bisect_right(_REGION_BASES, mcptr) - 1
        if i >= 0:
            r = _REGIONS[i]
            if r[0] <= mcptr < r[0] + r[1] and r[4]() is not None:
                _LAST_REGION = r
                return r
    return None


def _peer_stride(mcptr: int, world_size: int, nbytes: int) -> int:
    """Distance between the partial buffers that `mcptr` addresses, after checking that
    the `nbytes` the kernel reads from every slot lie inside the slot."""
    if world_size == 1:
        return 16  # unused: there is only partial 0
    r = _find_region(mcptr)
    if r is None:
        raise RuntimeError(
            f"mcptr 0x{mcptr:x} is not inside slot 0 of a registered partials region "
            "(allocate the staging buffers with tokenweave_amd.PartialsBuffer)")
    base, stride, slots, usable, _ = r
    _require(world_size <= slots,
             f"world_size {world_size} exceeds the {slots} slots of the partials region")
    if (mcptr - base) + nbytes > usable:
        raise RuntimeError(
            f"the rows of this call ({nbytes} bytes at offset {mcptr - base}) reach past the "
            f"{usable} usable bytes of a staging slot")
    return stride


# --- workspace of the split-row kernel (decode-size batches) -------------------
# One zeroed TW_SPLIT_WORKSPACE_BYTES buffer per (device, stream): calls on one stream
# are ordered, which is what sharing a workspace requires.  Allocated on the first
# small-batch call on that stream — never while the stream is being captured into a
# graph — and kept for the life of the process.
_SPLIT_WS: Dict[Tuple[int, int], torch.Tensor] = {}


def split_workspace(device_index: int, stream_ptr: int) -> Optional[torch.Tensor]:
    """The workspace of (device, stream), made on first use.  While the stream is being
    captured nothing is allocated (the buffer would come out of the graph's private pool
    and its fill kernel would be recorded): without a workspace made beforehand
    (`prepare_split_workspace`, or any eager decode-size call on that stream) the caller
    gets None and runs the one-workgroup-per-row kernel, whose results are the same bits."""
    ws = _SPLIT_WS.get((device_index, stream_ptr))
    if ws is None:
        if torch.cuda.is_current_stream_capturing():
            return None
        ws = torch.zeros(_lib.TW_SPLIT_WORKSPACE_BYTES, dtype=torch.uint8,
                         device=torch.device("cuda", device_index))
        assert ws.data_ptr() % 256 == 0
        _SPLIT_WS[(device_index, stream_ptr)] = ws
    return ws


def prepare_split_workspace(device=None, stream: Optional[torch.cuda.Stream] = None) -> None:
    """Create the split-row workspace of `stream` (default: the current stream of `device`)
    now.  Call it before capturing decode-size calls of `fused_rs_ln_ag_cta` /
    `fused_rs_ln_cta` / `reduce_add_rms_norm` on that stream into a HIP graph
    (`torch.cuda.graph(g, stream=stream)`): a capture never allocates, and without the
    workspace those calls record the one-workgroup-per-row kernel (same results, up to
    0.8 us slower per call).  A graph's split-row nodes use the capture stream's workspace:
    graphs captured on one stream must not be replayed concurrently on different streams."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    idx = dev.index if dev.index is not None else torch.cuda.current_device()
    if COMPILED_BINDING:
        with torch.cuda.device(idx), torch.cuda.stream(stream or torch.cuda.current_stream(idx)):
            _T.prepare_split_workspace(idx)
    sp = (stream or torch.cuda.current_stream(idx)).cuda_stream
    with torch.cuda.device(idx):
        split_workspace(idx, sp)


def _wants_split(T: int, cap: int) -> bool:
    """Whether an uncapped call of T rows goes through the workspace entry point: decode-size
    batches (split rows) and batches of a few more rows than compute units (mixed launch); the
    library decides which kernel runs, the workspace is only made available here."""
    return cap <= 0 and 0 < T <= 2 * _lib.TW_SPLIT_MAX_TOKENS


def _fused_rs_ln(entry: str, kname: str, input, residual, weight, mcptr, signal_pads, rank,
                 world_size, MAX_CTAS, epsilon) -> None:
    del signal_pads  # no peers, no signal pads on one GPU
    _require_bf16(kname, input)
    _check_tensor("input", input, torch.bfloat16, input.device)
    _check_tensor("residual", residual, torch.bfloat16, input.device)
    T, H = _rows(input)
    _require(residual.shape == input.shape, "input and residual must have the same shape")
    _check_weight(weight, H, torch.bfloat16, input.device)
    if not 0 <= rank < world_size:
        raise RuntimeError(f"Invalid rank {rank}, must be in [0, {world_size - 1}]")
    stride = _peer_stride(int(mcptr), int(world_size), T * H * 2)
    cap = _cap(MAX_CTAS)
    with _on_device(input):
        sp = _stream_ptr(input)
        ws = None
        if _wants_split(T, cap):
            idx = input.device.index
            ws = split_workspace(torch.cuda.current_device() if idx is None else idx, sp)
        if ws is not None:
            _lib.check(_lib.lib().tw_fused_rs_ln_ag_cta_ws(
                input.data_ptr(), residual.data_ptr(), weight.data_ptr(), int(mcptr), stride,
                int(rank), int(world_size), cap, epsilon, T, H, ws.data_ptr(), ws.numel(), sp))
            return
        _lib.check(getattr(_lib.lib(), entry)(
            input.data_ptr(), residual.data_ptr(), weight.data_ptr(), int(mcptr), stride,
            int(rank), int(world_size), cap, epsilon, T, H, sp))


def fused_rs_ln_ag_cta(input: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                       mcptr: int, signal_pads: int, rank: int, world_size: int, MAX_CTAS: int,
                       epsilon: float) -> None:
    _fused_rs_ln("tw_fused_rs_ln_ag_cta", "fused_rs_ln_ag_cta_kernel", input, residual, weight,
                 mcptr, signal_pads, rank, world_size, MAX_CTAS, epsilon)


def fused_rs_ln_cta(input: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                    mcptr: int, signal_pads: int, rank: int, world_size: int, MAX_CTAS: int,
                    epsilon: float) -> None:
    _fused_rs_ln("tw_fused_rs_ln_cta", "fused_rs_ln_cta_kernel", input, residual, weight,
                 mcptr, signal_pads, rank, world_size, MAX_CTAS, epsilon)


# ---------------------------------------------------------------------------
# one-GPU general form and the weave GEMM (no counterpart in vllm/_custom_ops.py)
# ---------------------------------------------------------------------------
class BoundOp:
    """An op whose arguments were checked once and frozen into one C-ABI call.

    `op()` enqueues it on the current stream of the tensors' device, `op(stream)` on
    the given `torch.cuda.Stream`: a single ctypes call, for loops where the regular
    shims' argument checks (several microseconds of Python) would outlast the kernel.
    The bound tensors are kept alive; their addresses and shapes must not change."""
    __slots__ = ("_fn", "_args", "_keep", "_device", "_index")

    def __init__(self, fn, args, keep, device):
        self._fn, self._args, self._keep, self._device = fn, args, keep, device
        self._index = device.index if device.index is not None else torch.cuda.current_device()

    def __call__(self, stream: Optional[torch.cuda.Stream] = None) -> None:
        if stream is not None:
            sp = stream.cuda_stream
        elif _raw_stream is not None:
            sp = _raw_stream(self._index)
        else:
            sp = torch.cuda.current_stream(self._device).cuda_stream
        cur = _raw_device() if _raw_device is not None else torch.cuda.current_device()
        if cur != self._index:
            with torch.cuda.device(self._index):
                rc = self._fn(*self._args, sp)
        else:
            rc = self._fn(*self._args, sp)
        if rc:
            _lib.check(rc)


def _check_reduce_add_rms_norm(partials, out, residual, weight, MAX_CTAS):
    """Argument checks of the pointer-list op; returns (ptrs, P, T, H, cap, device)."""
    P = len(partials)
    _require(1 <= P <= _lib.TW_MAX_PARTIALS,
             f"number of partials {P} not in [1, {_lib.TW_MAX_PARTIALS}]")
    _require_bf16("reduce_add_rms_norm_kernel", out)
    dev = out.device
    _check_tensor("out", out, torch.bfloat16, dev)
    _check_tensor("residual", residual, torch.bfloat16, dev)
    T, H = _rows(out)
    _require(residual.shape == out.shape, "out and residual must have the same shape")
    for i, p in enumerate(partials):
        if not (p.is_cuda and p.dtype == torch.bfloat16 and p.device == dev and p.is_contiguous()):
            _check_tensor(f"partials[{i}]", p, torch.bfloat16, dev)
        if p.shape != out.shape:
            raise RuntimeError(f"partials[{i}] has shape {tuple(p.shape)}, expected {tuple(out.shape)}")
    _check_weight(weight, H, torch.bfloat16, dev)
    ptrs = (ctypes.c_void_p * P)(*[p.data_ptr() for p in partials])
    return ptrs, P, T, H, _cap(MAX_CTAS), dev


def reduce_add_rms_norm(partials: Sequence[torch.Tensor], out: torch.Tensor,
                        residual: torch.Tensor, weight: torch.Tensor, epsilon: float,
                        MAX_CTAS: Optional[int] = None, split: Optional[bool] = None) -> None:
    """out <- RMSNorm(sum_p partials[p] + residual) * weight; residual <- the sum.
    `out` may be one of the partials.  Uncapped calls of at most TW_SPLIT_MAX_TOKENS rows
    go through the split-row entry point (several workgroups per row where that pays, same
    bits) with the workspace of the current stream; `split=False` forces the
    one-workgroup-per-row kernel."""
    ptrs, P, T, H, cap, dev = _check_reduce_add_rms_norm(partials, out, residual, weight, MAX_CTAS)
    L = _lib.lib()
    with _on_device(out):
        sp = _stream_ptr(out)
        ws = None
        if _wants_split(T, cap) if split is None else split:
            ws = split_workspace(dev.index if dev.index is not None else torch.cuda.current_device(), sp)
        if ws is not None:
            rc = L.tw_reduce_add_rms_norm_ws(ptrs, P, out.data_ptr(), residual.data_ptr(), weight.data_ptr(), T, H,
                                             cap, epsilon, ws.data_ptr(), ws.numel(), sp)
        else:
            rc = L.tw_reduce_add_rms_norm(ptrs, P, out.data_ptr(), residual.data_ptr(), weight.data_ptr(), T, H,
                                          cap, epsilon, sp)
    if rc:
        _lib.check(rc)


def bind_reduce_add_rms_norm(partials: Sequence[torch.Tensor], out: torch.Tensor,
                             residual: torch.Tensor, weight: torch.Tensor, epsilon: float,
                             MAX_CTAS: Optional[int] = None, split: Optional[bool] = None) -> BoundOp:
    """`reduce_add_rms_norm` with the checks done now and the launch deferred.  A bound op
    of a decode-size batch owns its split-row workspace: it may be launched on any stream,
    but not on two at once."""
    ptrs, P, T, H, cap, dev = _check_reduce_add_rms_norm(partials, out, residual, weight, MAX_CTAS)
    keep = [list(partials), out, residual, weight]
    args = (ptrs, P, out.data_ptr(), residual.data_ptr(), weight.data_ptr(), T, H, cap, epsilon)
    if _wants_split(T, cap) if split is None else split:
        ws = torch.zeros(_lib.TW_SPLIT_WORKSPACE_BYTES, dtype=torch.uint8, device=dev)
        keep.append(ws)
        return BoundOp(_lib.lib().tw_reduce_add_rms_norm_ws, args + (ws.data_ptr(), ws.numel()), keep, dev)
    return BoundOp(_lib.lib().tw_reduce_add_rms_norm, args, keep, dev)


def split_segments(num_tokens: int, hidden_size: int, MAX_CTAS: Optional[int] = None) -> int:
    """Workgroups per row the split-row entry points use for this shape on the current
    device (1 = one workgroup per row)."""
    return _lib.lib().tw_split_segments(num_tokens, hidden_size, _cap(MAX_CTAS))


# ---------------------------------------------------------------------------
# norm + static fp8 quantisation (vllm/_custom_ops.py rms_norm_static_fp8_quant /
# fused_add_rms_norm_static_fp8_quant -> csrc/layernorm_quant_kernels.cu)
# ---------------------------------------------------------------------------
FP8_DTYPE = torch.float8_e4m3fn  # gfx950 implements the OCP formats


def _check_fp8_out(out: torch.Tensor, like: torch.Tensor) -> None:
    if not (out.is_cuda and out.device == like.device):
        raise RuntimeError(f"result is on {out.device}, expected {like.device}")
    if out.dtype != FP8_DTYPE:
        raise NotImplementedError(f'"rms_norm_kernel_fp8_type" not implemented for \'{out.dtype}\'')
    _require(out.is_contiguous() and out.shape == like.shape,
             "result must be a contiguous fp8 tensor with the input's shape")


def _check_scale(scale: torch.Tensor, device) -> None:
    _require(isinstance(scale, torch.Tensor) and scale.is_cuda and scale.device == device,
             "scale must be a tensor on the input's device")
    _require(scale.dtype == torch.float32 and scale.numel() == 1, "scale must hold one float32 value")


def rms_norm_static_fp8_quant(result: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
                              scale: torch.Tensor, epsilon: float) -> None:
    code = _dtype_code("rms_norm_kernel_scalar_type", input)
    _check_tensor("input", input, input.dtype, input.device)
    _check_fp8_out(result, input)
    T, H = _rows(input)
    _check_weight(weight, H, input.dtype, input.device)
    _check_scale(scale, input.device)
    with _on_device(input):
        _lib.check(_lib.lib().tw_rms_norm_static_fp8_quant(
            result.data_ptr(), input.data_ptr(), weight.data_ptr(), scale.data_ptr(), T, H, epsilon,
            code, _stream_ptr(input)))


def fused_add_rms_norm_static_fp8_quant(result: torch.Tensor, input: torch.Tensor,
                                        residual: torch.Tensor, weight: torch.Tensor,
                                        scale: torch.Tensor, epsilon: float) -> None:
    code = _dtype_code("fused_add_rms_norm_kernel_scalar_type", input)
    _check_tensor("input", input, input.dtype, input.device)
    _check_tensor("residual", residual, input.dtype, input.device)
    _check_fp8_out(result, input)
    T, H = _rows(input)
    _require(residual.shape == input.shape, "input and residual must have the same shape")
    _check_weight(weight, H, input.dtype, input.device)
    _check_scale(scale, input.device)
    with _on_device(input):
        _lib.check(_lib.lib().tw_fused_add_rms_norm_static_fp8_quant(
            result.data_ptr(), input.data_ptr(), residual.data_ptr(), weight.data_ptr(),
            scale.data_ptr(), T, H, epsilon, code, _stream_ptr(input)))


def reduce_add_rms_norm_static_fp8_quant(partials: Sequence[torch.Tensor], result: torch.Tensor,
                                         residual: torch.Tensor, weight: torch.Tensor,
                                         scale: torch.Tensor, epsilon: float,
                                         MAX_CTAS: Optional[int] = None) -> None:
    """result(fp8) <- quantised RMSNorm(sum_p partials[p] + residual) * weight; residual <- the sum."""
    P = len(partials)
    _require(1 <= P <= _lib.TW_MAX_PARTIALS,
             f"number of partials {P} not in [1, {_lib.TW_MAX_PARTIALS}]")
    _require_bf16("reduce_add_rms_norm_kernel", residual)
    dev = residual.device
    _check_tensor("residual", residual, torch.bfloat16, dev)
    _check_fp8_out(result, residual)
    T, H = _rows(residual)
    for i, p in enumerate(partials):
        if not (p.is_cuda and p.dtype == torch.bfloat16 and p.device == dev and p.is_contiguous()):
            _check_tensor(f"partials[{i}]", p, torch.bfloat16, dev)
        _require(p.shape == residual.shape,
                 f"partials[{i}] has shape {tuple(p.shape)}, expected {tuple(residual.shape)}")
    _check_weight(weight, H, torch.bfloat16, dev)
    _check_scale(scale, dev)
    ptrs = (ctypes.c_void_p * P)(*[p.data_ptr() for p in partials])
    with _on_device(residual):
        _lib.check(_lib.lib().tw_reduce_add_rms_norm_static_fp8_quant(
            ptrs, P, result.data_ptr(), residual.data_ptr(), weight.data_ptr(), scale.data_ptr(), T, H,
            _cap(MAX_CTAS), epsilon, _stream_ptr(residual)))


# ---------------------------------------------------------------------------
# norm + dynamic per-token quantisation (vllm/_custom_ops.py:256-272 ->
# csrc/quantization/fused_kernels/fused_layernorm_dynamic_per_token_quant.cu)
# ---------------------------------------------------------------------------
QUANT_FP8_E4M3FN, QUANT_INT8 = 0, 1


def _check_dyn_quant(result, like, scales, scale_ub, T):
    """The launcher's checks (fused_layernorm_dynamic_per_token_quant.cu:139-147)."""
    _require(result.is_cuda and result.device == like.device,
             f"result is on {result.device}, expected {like.device}")
    _require(result.dtype in (FP8_DTYPE, torch.int8),
             f"result must be {FP8_DTYPE} or torch.int8, got {result.dtype}")
    _require(result.is_contiguous() and result.shape == like.shape,
             "result must be contiguous and have the input's shape")
    _require(scales.is_cuda and scales.device == like.device and scales.dtype == torch.float32,
             "scales must be a float32 tensor on the input's device")
    if not (scales.is_contiguous() and scales.numel() == T):
        raise RuntimeError(f"scales must hold {T} contiguous values")
    if scale_ub is not None:
        _require(result.dtype == FP8_DTYPE, "scale_ub is defined for fp8 output only")
        _check_scale(scale_ub, like.device)
    return QUANT_FP8_E4M3FN if result.dtype == FP8_DTYPE else QUANT_INT8


def rms_norm_dynamic_per_token_quant_out(result: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
                                         scale: torch.Tensor, epsilon: float,
                                         scale_ub: Optional[torch.Tensor] = None,
                                         residual: Optional[torch.Tensor] = None) -> None:
    """The registered op (schema csrc/torch_bindings.cpp:216-219): result, scale and
    residual are written in place."""
    code = _dtype_code("rms_norm_dynamic_per_token_quant_dispatch", input)
    _check_tensor("input", input, input.dtype, input.device)
    T, H = _rows(input)
    kind = _check_dyn_quant(result, input, scale, scale_ub, T)
    _check_weight(weight, H, input.dtype, input.device)
    if residual is not None:
        _check_tensor("residual", residual, input.dtype, input.device)
        _require(residual.shape == input.shape, "input and residual must have the same shape")
    with _on_device(input):
        _lib.check(_lib.lib().tw_rms_norm_dynamic_per_token_quant(
            result.data_ptr(), input.data_ptr(), weight.data_ptr(), scale.data_ptr(),
            scale_ub.data_ptr() if scale_ub is not None else None,
            residual.data_ptr() if residual is not None else None, T, H, epsilon, code, kind,
            _stream_ptr(input)))


def rms_norm_dynamic_per_token_quant(input: torch.Tensor, weight: torch.Tensor, epsilon: float,
                                     quant_dtype: torch.dtype,
                                     scale_ub: Optional[torch.Tensor] = None,
                                     residual: Optional[torch.Tensor] = None):
    """vllm/_custom_ops.py:256-272: allocates the outputs, returns (output, scales);
    residual (if given) is updated in place."""
    output = torch.empty_like(input, dtype=quant_dtype)
    scales = torch.empty((input.numel() // input.shape[-1], 1), device=input.device, dtype=torch.float32)
    rms_norm_dynamic_per_token_quant_out(output, input, weight, scales, epsilon, scale_ub, residual)
    return output, scales


def reduce_add_rms_norm_dynamic_per_token_quant(partials: Sequence[torch.Tensor], result: torch.Tensor,
                                                scales: torch.Tensor, residual: Optional[torch.Tensor],
                                                weight: torch.Tensor, epsilon: float,
                                                scale_ub: Optional[torch.Tensor] = None,
                                                MAX_CTAS: Optional[int] = None) -> None:
    """result <- dynamic per-token quantisation of RMSNorm(sum_p partials[p] + residual) * weight,
    scales <- the row scales, residual <- the sum (when given)."""
    P = len(partials)
    _require(1 <= P <= _lib.TW_MAX_PARTIALS,
             f"number of partials {P} not in [1, {_lib.TW_MAX_PARTIALS}]")
    first = partials[0]
    _require_bf16("reduce_add_rms_norm_kernel", first)
    dev = first.device
    T, H = _rows(first)
    for i, p in enumerate(partials):
        if not (p.is_cuda and p.dtype == torch.bfloat16 and p.device == dev and p.is_contiguous()):
            _check_tensor(f"partials[{i}]", p, torch.bfloat16, dev)
        if p.shape != first.shape:
            raise RuntimeError(f"partials[{i}] has shape {tuple(p.shape)}, expected {tuple(first.shape)}")
    if residual is not None:
        _check_tensor("residual", residual, torch.bfloat16, dev)
        _require(residual.shape == first.shape, "partials and residual must have the same shape")
    kind = _check_dyn_quant(result, first, scales, scale_ub, T)
    _check_weight(weight, H, torch.bfloat16, dev)
    ptrs = (ctypes.c_void_p * P)(*[p.data_ptr() for p in partials])
    with _on_device(first):
        _lib.check(_lib.lib().tw_reduce_add_rms_norm_dynamic_per_token_quant(
            ptrs, P, result.data_ptr(), scales.data_ptr(),
            residual.data_ptr() if residual is not None else None, weight.data_ptr(),
            scale_ub.data_ptr() if scale_ub is not None else None, T, H, _cap(MAX_CTAS), epsilon, kind,
            _stream_ptr(first)))


def _check_bias(bias, N, dev):
    if bias is None:
        return
    _check_tensor("bias", bias, torch.bfloat16, dev)
    _require(bias.dim() == 1 and bias.numel() == N, f"bias has shape {tuple(bias.shape)}, expected {(N,)}")


def _prepare_gemm_bf16_nt(out, a, b, max_cus, bias=None):
    _require_bf16("gemm_bf16_nt_kernel", a)
    dev = a.device
    _check_tensor("a", a, torch.bfloat16, dev)
    _check_tensor("b", b, torch.bfloat16, dev)
    _require(a.dim() == 2 and b.dim() == 2 and out.dim() == 2, "gemm operands must be 2-D")
    _require(out.is_cuda and out.device == dev and out.dtype == torch.bfloat16,
             "out must be a bf16 tensor on the same device")
    M, K = a.shape
    N, K2 = b.shape
    _require(K == K2, f"inner dimensions differ: a is {tuple(a.shape)}, b is {tuple(b.shape)}")
    _require(tuple(out.shape) == (M, N), f"out has shape {tuple(out.shape)}, expected {(M, N)}")
    _require(out.stride(1) == 1 and (M <= 1 or out.stride(0) >= N), "out rows must be contiguous")
    _check_bias(bias, N, dev)
    ldc = out.stride(0) if M > 1 else max(N, out.stride(0))
    if bias is None:
        args = (out.data_ptr(), a.data_ptr(), b.data_ptr(), M, N, K, ldc, _cap(max_cus))
        return _lib.lib().tw_gemm_bf16_nt, args, (out, a, b), dev
    args = (out.data_ptr(), a.data_ptr(), b.data_ptr(), bias.data_ptr(), M, N, K, ldc, _cap(max_cus))
    return _lib.lib().tw_gemm_bf16_nt_bias, args, (out, a, b, bias), dev


def gemm_bf16_nt(out: torch.Tensor, a: torch.Tensor, b: torch.Tensor,
                 max_cus: Optional[int] = None, bias: Optional[torch.Tensor] = None) -> None:
    """out[M, N] <- a[M, K] @ b[N, K]^T (bf16, fp32 accumulate), then `out += bias` as the
    reference does it (on the rounded product, rounded again).  `out` may be a row slice of
    a wider buffer (row stride >= N).  The in-place row-parallel linear of
    vllm/model_executor/layers/linear.py:203-228."""
    BoundOp(*_prepare_gemm_bf16_nt(out, a, b, max_cus, bias))()


def bind_gemm_bf16_nt(out: torch.Tensor, a: torch.Tensor, b: torch.Tensor,
                      max_cus: Optional[int] = None, bias: Optional[torch.Tensor] = None) -> BoundOp:
    """`gemm_bf16_nt` with the checks done now and the launch deferred."""
    return BoundOp(*_prepare_gemm_bf16_nt(out, a, b, max_cus, bias))


def _prepare_gemm_bf16_nt_partials(outs, a_list, b_list, max_cus, biases=None):
    P = len(outs)
    _require(1 <= P <= _lib.TW_MAX_PARTIALS, f"number of partials {P} not in [1, {_lib.TW_MAX_PARTIALS}]")
    _require(len(a_list) == P and len(b_list) == P, "outs, a and b must have one entry per partial")
    _require(biases is None or len(biases) == P, "biases must have one entry (a tensor or None) per partial")
    shape = None
    for p in range(P):
        # the per-product checks of gemm_bf16_nt; all products must share one shape and row stride
        _, args, _, dev = _prepare_gemm_bf16_nt(outs[p], a_list[p], b_list[p], max_cus,
                                                None if biases is None else biases[p])
        dims = args[-5:-1]
        if shape is None:
            shape, dev0 = dims, dev
        _require(dims == shape and dev == dev0,
                 f"partial {p} has (M, N, K, row stride) {dims}, partial 0 has {shape}")
    vp = ctypes.c_void_p
    o = (vp * P)(*[t.data_ptr() for t in outs])
    a = (vp * P)(*[t.data_ptr() for t in a_list])
    b = (vp * P)(*[t.data_ptr() for t in b_list])
    keep = (list(outs), list(a_list), list(b_list))
    if biases is None or all(t is None for t in biases):
        return _lib.lib().tw_gemm_bf16_nt_partials, (o, a, b, P, *shape, _cap(max_cus)), keep, dev0
    bs = (vp * P)(*[None if t is None else t.data_ptr() for t in biases])
    return (_lib.lib().tw_gemm_bf16_nt_partials_bias, (o, a, b, bs, P, *shape, _cap(max_cus)),
            keep + (list(biases),), dev0)


def gemm_bf16_nt_partials(outs: Sequence[torch.Tensor], a: Sequence[torch.Tensor], b: Sequence[torch.Tensor],
                          max_cus: Optional[int] = None,
                          biases: Optional[Sequence[Optional[torch.Tensor]]] = None) -> None:
    """outs[p][M, N] <- a[p][M, K] @ b[p][N, K]^T (+ biases[p] where given) for every p in ONE
    launch: the P row-parallel partial sums of a token split, each written straight into its
    rank's staging rows (`outs[p]` = `PartialsBuffer.slot(p)[first_row:first_row + M]`).  The
    producer side of the fused op: vllm/model_executor/layers/linear.py:203-228, 1310-1321
    (only rank 0 adds its bias, :1306-1308: pass it as biases[0], None elsewhere)."""
    BoundOp(*_prepare_gemm_bf16_nt_partials(outs, a, b, max_cus, biases))()


def bind_gemm_bf16_nt_partials(outs: Sequence[torch.Tensor], a: Sequence[torch.Tensor],
                               b: Sequence[torch.Tensor], max_cus: Optional[int] = None,
                               biases: Optional[Sequence[Optional[torch.Tensor]]] = None) -> BoundOp:
    """`gemm_bf16_nt_partials` with the checks done now and the launch deferred."""
    return BoundOp(*_prepare_gemm_bf16_nt_partials(outs, a, b, max_cus, biases))


def num_compute_units(device=None) -> int:
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    with torch.cuda.device(dev):
        n = _lib.lib().tw_num_compute_units()
    _require(n > 0, "could not query the device's compute-unit count")
    return n


# ---------------------------------------------------------------------------
# torch.library registration: the reference's schema strings
# (csrc/torch_bindings.cpp:135-171), namespace `tokenweave_amd`.
# ---------------------------------------------------------------------------
SCHEMAS = {
    "rms_norm": "rms_norm(Tensor! result, Tensor input, Tensor weight, float epsilon) -> ()",
    "fused_add_rms_norm":
        "fused_add_rms_norm(Tensor! input, Tensor! residual, Tensor weight, float epsilon) -> ()",
    "rms_norm_inplace":
        "rms_norm_inplace(Tensor! result, Tensor! input, Tensor weight, float epsilon) -> ()",
    "fused_rs_ln_ag_cta":
        "fused_rs_ln_ag_cta(Tensor! input, Tensor! residual, Tensor weight, int mcptr, "
        "int signal_pads, int rank, int world_size, int MAX_CTAS, float epsilon) -> ()",
    "fused_add_rms_norm_cta":
        "fused_add_rms_norm_cta(Tensor! input, Tensor! residual, Tensor weight, int MAX_CTAS, "
        "float epsilon) -> ()",
    "fused_rs_ln_cta":
        "fused_rs_ln_cta(Tensor! input, Tensor! residual, Tensor weight, int mcptr, "
        "int signal_pads, int rank, int world_size, int MAX_CTAS, float epsilon) -> ()",
    # csrc/torch_bindings.cpp:199-213
    "rms_norm_static_fp8_quant":
        "rms_norm_static_fp8_quant(Tensor! result, Tensor input, Tensor weight, Tensor scale, "
        "float epsilon) -> ()",
    "fused_add_rms_norm_static_fp8_quant":
        "fused_add_rms_norm_static_fp8_quant(Tensor! result, Tensor input, Tensor! residual, "
        "Tensor weight, Tensor scale, float epsilon) -> ()",
    # csrc/torch_bindings.cpp:216-219
    "rms_norm_dynamic_per_token_quant":
        "rms_norm_dynamic_per_token_quant(Tensor! result, Tensor input, Tensor weight, Tensor! scale, "
        "float epsilon, Tensor? scale_ub, Tensor!? residual) -> ()",
}

_IMPLS = {
    "rms_norm": rms_norm,
    "fused_add_rms_norm": fused_add_rms_norm,
    "rms_norm_inplace": rms_norm_inplace,
    "fused_rs_ln_ag_cta": fused_rs_ln_ag_cta,
    "fused_add_rms_norm_cta": fused_add_rms_norm_cta,
    "fused_rs_ln_cta": fused_rs_ln_cta,
    "rms_norm_static_fp8_quant": rms_norm_static_fp8_quant,
    "fused_add_rms_norm_static_fp8_quant": fused_add_rms_norm_static_fp8_quant,
    "rms_norm_dynamic_per_token_quant": rms_norm_dynamic_per_token_quant_out,
}


def _no_cpu(name):
    def impl(*args, **kwargs):
        raise RuntimeError(f"tokenweave_amd::{name} has no CPU implementation; "
                           "pass tensors that live on the MI355X")
    return impl


via_ctypes = types.SimpleNamespace(
    rms_norm=rms_norm, fused_add_rms_norm=fused_add_rms_norm, rms_norm_inplace=rms_norm_inplace,
    fused_rs_ln_ag_cta=fused_rs_ln_ag_cta, fused_add_rms_norm_cta=fused_add_rms_norm_cta,
    fused_rs_ln_cta=fused_rs_ln_cta, rms_norm_static_fp8_quant=rms_norm_static_fp8_quant,
    fused_add_rms_norm_static_fp8_quant=fused_add_rms_norm_static_fp8_quant,
    rms_norm_dynamic_per_token_quant_out=rms_norm_dynamic_per_token_quant_out)

if COMPILED_BINDING:
    # One dispatcher call per op (the overload is resolved once, here); the argument
    # checks and the launch are the binding's.
    _op_rms_norm = _T.rms_norm.default
    _op_fused_add_rms_norm = _T.fused_add_rms_norm.default
    _op_rms_norm_inplace = _T.rms_norm_inplace.default
    _op_fused_add_rms_norm_cta = _T.fused_add_rms_norm_cta.default
    _op_fused_rs_ln_ag_cta = _T.fused_rs_ln_ag_cta.default
    _op_fused_rs_ln_cta = _T.fused_rs_ln_cta.default
    _op_rms_norm_static_fp8_quant = _T.rms_norm_static_fp8_quant.default
    _op_fused_add_rms_norm_static_fp8_quant = _T.fused_add_rms_norm_static_fp8_quant.default
    _op_rms_norm_dynamic_per_token_quant = _T.rms_norm_dynamic_per_token_quant.default

    def rms_norm(out: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,  # noqa: F811
                 epsilon: float) -> None:
        _op_rms_norm(out, input, weight, epsilon)

    def fused_add_rms_norm(input: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,  # noqa: F811
                           epsilon: float) -> None:
        _op_fused_add_rms_norm(input, residual, weight, epsilon)

    def rms_norm_inplace(out: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,  # noqa: F811
                         epsilon: float) -> None:
        _op_rms_norm_inplace(out, input, weight, epsilon)

    def fused_add_rms_norm_cta(input: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,  # noqa: F811
                               MAX_CTAS: int, epsilon: float) -> None:
        _op_fused_add_rms_norm_cta(input, residual, weight, 0 if MAX_CTAS is None else MAX_CTAS, epsilon)

    def fused_rs_ln_ag_cta(input: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,  # noqa: F811
                           mcptr: int, signal_pads: int, rank: int, world_size: int, MAX_CTAS: int,
                           epsilon: float) -> None:
        _op_fused_rs_ln_ag_cta(input, residual, weight, mcptr, signal_pads, rank, world_size,
                               0 if MAX_CTAS is None else MAX_CTAS, epsilon)

    def fused_rs_ln_cta(input: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,  # noqa: F811
                        mcptr: int, signal_pads: int, rank: int, world_size: int, MAX_CTAS: int,
                        epsilon: float) -> None:
        _op_fused_rs_ln_cta(input, residual, weight, mcptr, signal_pads, rank, world_size,
                            0 if MAX_CTAS is None else MAX_CTAS, epsilon)

    def rms_norm_static_fp8_quant(result: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,  # noqa: F811
                                  scale: torch.Tensor, epsilon: float) -> None:
        _op_rms_norm_static_fp8_quant(result, input, weight, scale, epsilon)

    def fused_add_rms_norm_static_fp8_quant(result: torch.Tensor, input: torch.Tensor,  # noqa: F811
                                            residual: torch.Tensor, weight: torch.Tensor,
                                            scale: torch.Tensor, epsilon: float) -> None:
        _op_fused_add_rms_norm_static_fp8_quant(result, input, residual, weight, scale, epsilon)

    def rms_norm_dynamic_per_token_quant_out(result: torch.Tensor, input: torch.Tensor,  # noqa: F811
                                             weight: torch.Tensor, scale: torch.Tensor, epsilon: float,
                                             scale_ub: Optional[torch.Tensor] = None,
                                             residual: Optional[torch.Tensor] = None) -> None:
        """The registered op (schema csrc/torch_bindings.cpp:216-219): result, scale and
        residual are written in place."""
        _op_rms_norm_dynamic_per_token_quant(result, input, weight, scale, epsilon, scale_ub, residual)
else:
    _library = torch.library.Library("tokenweave_amd", "DEF")
    for _name, _schema in SCHEMAS.items():
        _library.define(_schema)
        _library.impl(_name, _IMPLS[_name], "CUDA")
        _library.impl(_name, _no_cpu(_name), "CPU")
