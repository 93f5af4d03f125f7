"""ctypes binding of libsba.so (the C ABI declared in include/sba.h).

This is the only place that touches the shared library.  There is no fallback: if the library has not
been built, or a call reports an error, the operators raise.
"""
from __future__ import annotations

import ctypes
import math
import os
from typing import Optional

import torch

from .utils import custom_op

_LIB_NAME = "libsba.so"
ABI_VERSION = 5          # SBA_VERSION of include/sba.h this binding mirrors
_lib = None
# Optional ctypes array of hipEvent_t handed to the next calls as SbaArgs.trace_events (benchmarks only).
TRACE_EVENTS = None

SBA_BF16, SBA_F32, SBA_F16 = 0, 1, 2
_DTYPES = {torch.bfloat16: SBA_BF16, torch.float32: SBA_F32, torch.float16: SBA_F16}


class SbaTensor(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("stride_batch", ctypes.c_int64), ("stride_head", ctypes.c_int64),
                ("stride_token", ctypes.c_int64)]


class SbaVector(ctypes.Structure):
    _fields_ = SbaTensor._fields_


class SbaArgs(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int32), ("head_dim", ctypes.c_int32), ("num_heads", ctypes.c_int32), ("num_seqs", ctypes.c_int32),
        ("total_tokens", ctypes.c_int64), ("max_seqlen", ctypes.c_int64),
        ("logit_scale", ctypes.c_float), ("attend_current", ctypes.c_int32),
        ("cu_seqlens", ctypes.c_void_p), ("cu_is_int64", ctypes.c_int32), ("cu_has_leading_zero", ctypes.c_int32),
        ("q", SbaTensor), ("k", SbaTensor), ("v", SbaTensor), ("o", SbaTensor),
        ("rem", SbaVector), ("row_stat", ctypes.c_void_p), ("carry", ctypes.c_void_p),
        ("d_o", SbaTensor), ("d_rem", SbaVector), ("dq", SbaTensor), ("dk", SbaTensor), ("dv", SbaTensor),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t), ("stream", ctypes.c_void_p),
        ("trace_events", ctypes.POINTER(ctypes.c_void_p)),
        ("add_remainder", ctypes.c_int32), ("recompute_carry", ctypes.c_int32), ("carry_slots", ctypes.c_int64),
        ("backward_kernels", ctypes.c_int32), ("reserved0", ctypes.c_int32),
    ]


class SbaPlan(ctypes.Structure):
    _fields_ = [("status", ctypes.c_int32), ("longest", ctypes.c_int32), ("covered_tokens", ctypes.c_int64),
                ("query_tiles", ctypes.c_int64), ("key_tiles", ctypes.c_int64), ("carry_slots", ctypes.c_int64),
                ("pairs", ctypes.c_int64)]


EXPORTS = ("sba_version", "sba_strerror", "sba_workspace_bytes", "sba_plan_host", "sba_fwd", "sba_fwd_static", "sba_bwd", "sba_bwd_kernels")
STATUS_OFFSET = 8        # SBA_STATUS_OFFSET: the scheduler's status word inside the workspace
# Debugging aid for the tests: fill the carry buffer and the workspaces with NaN bit patterns before every launch,
# so that a kernel reading a slot nobody wrote shows up as NaN instead of passing on whatever the allocator returned.
POISON = os.environ.get("SBA_DEBUG_POISON", "0") == "1"
# Read the scheduler's status word back after every launch (one device-to-host copy and a synchronisation per call)
# and raise on a schedule the device refused.  Without it a bad ``cu_seqlens`` that only exists on the device yields
# all-zero outputs and gradients and no error.
DEBUG_CHECK = os.environ.get("SBA_DEBUG_CHECK", "0") == "1"
# SbaArgs.backward_kernels: 0 = the library chooses, 1 = dQ then dK/dV, 2 = one chained kernel where it applies.
BACKWARD_KERNELS = int(os.environ.get("SBA_BACKWARD_KERNELS", "0"))
# Attention kernels the last traced backward ran: 1 (chained) or 2 (set when TRACE_EVENTS is).
LAST_BWD_KERNELS = 0
_STATUS_TEXT = {1: "cu_seqlens is not a non-decreasing sequence within [0, total_tokens] (or its leading entry is not 0)",
                2: "the carry buffer is too small for these sequence lengths (max_seqlens understated?)",
                3: "one-kernel backward: a workgroup gave up waiting for the key tile below its own",
                4: "one-kernel backward: the workgroups of a head did not share an XCD"}


def check_status(ws: torch.Tensor, what: str):
    """Raise if the device-side scheduler (or the chained backward) left a non-zero status word in ``ws``."""
    status = int(ws[STATUS_OFFSET:STATUS_OFFSET + 4].view(torch.int32).item())
    if status != 0:
        raise ValueError(f"{what}: {_STATUS_TEXT.get(status, 'status %d' % status)}; outputs of this call are not valid")


def library_path() -> str:
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), _LIB_NAME)


def lib():
    """Load libsba.so once.  Raises if it has not been built (run `make -C csrc` or __graft_entry__.build())."""
    global _lib
    if _lib is None:
        path = library_path()
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: build it with `make -C stickbreaking-attention_amd/csrc`; "
                               "stick-breaking attention has no fallback path")
        handle = ctypes.CDLL(path)
        handle.sba_version.restype = ctypes.c_int
        handle.sba_strerror.restype = ctypes.c_char_p
        handle.sba_strerror.argtypes = [ctypes.c_int]
        handle.sba_workspace_bytes.restype = ctypes.c_int
        handle.sba_workspace_bytes.argtypes = [ctypes.POINTER(SbaArgs)] + [ctypes.POINTER(ctypes.c_size_t)] * 3
        handle.sba_plan_host.restype = ctypes.c_int
        handle.sba_plan_host.argtypes = [ctypes.POINTER(SbaArgs), ctypes.c_void_p, ctypes.POINTER(SbaPlan)]
        for name in ("sba_fwd", "sba_fwd_static", "sba_bwd", "sba_bwd_kernels"):
            fn = getattr(handle, name)
            fn.restype = ctypes.c_int
            fn.argtypes = [ctypes.POINTER(SbaArgs)]
        if handle.sba_version() != ABI_VERSION:
            raise RuntimeError(f"{path}: ABI version {handle.sba_version()} != {ABI_VERSION}")
        _lib = handle
    return _lib


def _check(status: int, what: str):
    if status != 0:
        raise RuntimeError(f"{what} failed: {lib().sba_strerror(status).decode()} (status {status})")


def _tensor(t: Optional[torch.Tensor], fixed: bool) -> SbaTensor:
    if t is None:
        return SbaTensor(None, 0, 0, 0)
    if fixed:
        return SbaTensor(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))
    return SbaTensor(t.data_ptr(), 0, t.stride(0), t.stride(1))


def _vector(t: Optional[torch.Tensor], fixed: bool) -> SbaVector:
    if t is None:
        return SbaVector(None, 0, 0, 0)
    if fixed:
        return SbaVector(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))
    return SbaVector(t.data_ptr(), 0, t.stride(0), t.stride(1))


def rows_contiguous(t: torch.Tensor) -> torch.Tensor:
    """The kernels need unit stride along head_dim (as the reference does, sb_varlen_fwd.py:235)."""
    return t if t.stride(-1) == 1 else t.contiguous()


def _require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("stick-breaking attention runs on the GPU only (got a CPU tensor); there is no CPU path")


def plan_host(cu_seqlens_host: Optional[torch.Tensor], cu_has_leading_zero: bool, total_tokens: int,
              num_seqs: Optional[int] = None, attend_current: bool = False) -> SbaPlan:
    """What the device scheduler will derive from ``cu_seqlens``, computed by the library on the host from a host
    copy (sba_plan_host): validity, tile counts, the exact number of carry slots per head, visible pairs."""
    a = SbaArgs()
    a.total_tokens = int(total_tokens)
    a.attend_current = 1 if attend_current else 0
    ptr = None
    if cu_seqlens_host is not None:
        assert cu_seqlens_host.device.type == "cpu"
        if cu_seqlens_host.dtype not in (torch.int32, torch.int64):
            cu_seqlens_host = cu_seqlens_host.to(torch.int64)
        cu_seqlens_host = cu_seqlens_host.contiguous()
        a.num_seqs = cu_seqlens_host.numel() - (1 if cu_has_leading_zero else 0)
        a.cu_is_int64 = 1 if cu_seqlens_host.dtype == torch.int64 else 0
        a.cu_has_leading_zero = 1 if cu_has_leading_zero else 0
        ptr = cu_seqlens_host.data_ptr()
    else:
        a.num_seqs = int(num_seqs)
    out = SbaPlan()
    _check(lib().sba_plan_host(ctypes.byref(a), ptr, ctypes.byref(out)), "sba_plan_host")
    return out


def _base_args(q, cu_seqlens, cu_has_leading_zero, max_seqlen, logit_scale, attend_current, carry_slots=0) -> SbaArgs:
    if q.dtype not in _DTYPES:
        raise TypeError(f"unsupported dtype {q.dtype}")
    a = SbaArgs()
    a.dtype = _DTYPES[q.dtype]
    fixed = cu_seqlens is None
    if fixed:
        B, H, L, D = q.shape
        a.num_seqs, a.num_heads, a.total_tokens, a.head_dim = B, H, L, D
        a.cu_seqlens = None
    else:
        H, T, D = q.shape
        a.num_heads, a.total_tokens, a.head_dim = H, T, D
        a.num_seqs = cu_seqlens.numel() - (1 if cu_has_leading_zero else 0)
        a.cu_seqlens = cu_seqlens.data_ptr()
        a.cu_is_int64 = 1 if cu_seqlens.dtype == torch.int64 else 0
        a.cu_has_leading_zero = 1 if cu_has_leading_zero else 0
    a.max_seqlen = int(max_seqlen) if max_seqlen else 0
    a.carry_slots = int(carry_slots) if (carry_slots and not fixed) else 0
    a.logit_scale = float(logit_scale)
    a.attend_current = 1 if attend_current else 0
    a.stream = torch.cuda.current_stream(q.device).cuda_stream
    a.backward_kernels = BACKWARD_KERNELS
    if TRACE_EVENTS is not None:
        a.trace_events = ctypes.cast(TRACE_EVENTS, ctypes.POINTER(ctypes.c_void_p))
    return a


def prepare_cu_seqlens(cu_seqlens: torch.Tensor, device) -> torch.Tensor:
    if cu_seqlens.dtype not in (torch.int32, torch.int64):
        cu_seqlens = cu_seqlens.to(torch.int64)
    if cu_seqlens.device != device:
        cu_seqlens = cu_seqlens.to(device)
    return cu_seqlens.contiguous()


def carry_elems(num_heads: int, total_tokens: int, num_seqs: int, max_seqlen, fixed: bool, carry_slots: int = 0) -> int:
    """fp32 elements of the ``carry`` buffer the forward fills for the backward: what the library reports
    through ``sba_workspace_bytes`` (one value per query row and 32-key sub-tile the row sweeps), computed
    here from shapes alone so that it can be traced by torch.compile.  ``carry_slots`` > 0 is the exact
    per-head count from ``plan_host``; otherwise packed batches use the bound T * max_seqlen / 64."""
    T, B = total_tokens, num_seqs
    if fixed:
        m = -(-T // 128)
        slots = B * 256 * m * (m + 1)
    elif carry_slots:
        slots = carry_slots
    else:
        max_len = max_seqlen if (max_seqlen and 0 < max_seqlen < T) else T
        slots = -(-(T * max_len) // 64) + 6 * T + 512 * B
    nbytes = -(-(slots * num_heads * 4) // 256) * 256
    return nbytes // 4


# Upper limit in bytes for the backward's workspace (None: whatever the whole call needs).  With a limit the library
# takes the heads through in groups that fit, one group after the other; together with ``save_carry=False`` this bounds
# the memory of a long-context backward by the planes of one group of heads.
BWD_WORKSPACE_LIMIT: Optional[int] = None


def set_backward_workspace_limit(nbytes: Optional[int]):
    global BWD_WORKSPACE_LIMIT
    BWD_WORKSPACE_LIMIT = None if nbytes is None else int(nbytes)


def _poison(t: torch.Tensor):
    t.view(torch.uint8).fill_(0xFF)          # every fp32 / 16-bit word becomes a NaN pattern, every int32 becomes -1


# Workspace sizes depend on the shape and the flags of a call only (never on pointers or on the lengths behind
# cu_seqlens), so they are asked for once per distinct call and remembered.
_WS_BYTES = {}


def _workspace_bytes(a: SbaArgs):
    """(forward workspace, backward workspace, carry) sizes in bytes for these arguments."""
    key = (a.dtype, a.num_heads, a.head_dim, a.num_seqs, a.total_tokens, a.max_seqlen, bool(a.cu_seqlens), a.cu_is_int64,
           a.cu_has_leading_zero, a.attend_current, a.add_remainder, a.recompute_carry, a.carry_slots, a.backward_kernels)
    got = _WS_BYTES.get(key)
    if got is None:
        f, b, c = ctypes.c_size_t(0), ctypes.c_size_t(0), ctypes.c_size_t(0)
        _check(lib().sba_workspace_bytes(ctypes.byref(a), ctypes.byref(f), ctypes.byref(b), ctypes.byref(c)), "sba_workspace_bytes")
        got = _WS_BYTES[key] = (f.value, b.value, c.value)
    return got


def _launch_fwd(q, k, v, cu_seqlens, cu_has_leading_zero, max_seqlen, carry_slots, logit_scale, attend_current, add_remainder,
                o, rem, neg_log_acc, carry):
    fixed = cu_seqlens is None
    with torch.cuda.device(q.device):
        a = _base_args(q, cu_seqlens, cu_has_leading_zero, max_seqlen, logit_scale, attend_current, carry_slots)
        a.add_remainder = 1 if add_remainder else 0
        a.q, a.k, a.v, a.o = (_tensor(t, fixed) for t in (q, k, v, o))
        a.rem = _vector(rem, fixed)
        a.row_stat = neg_log_acc.data_ptr()
        if carry.numel() == 0 and q.dtype != torch.float32:
            # no products kept: a backward, if one follows, rebuilds them, and the forward's scheduler checks their
            # capacity as that backward's will (both passes void, or neither)
            a.recompute_carry = 1
        need_fwd, _, need_carry_bytes = _workspace_bytes(a)
        ws = torch.empty(need_fwd, dtype=torch.uint8, device=q.device)
        a.workspace, a.workspace_bytes = ws.data_ptr(), need_fwd
        if POISON:
            _poison(ws)
            if carry.numel() > 0:
                _poison(carry)
        if carry.numel() > 0:
            if carry.numel() * 4 < need_carry_bytes:
                raise RuntimeError(f"carry buffer too small: {carry.numel() * 4} < {need_carry_bytes} bytes")
            a.carry = carry.data_ptr()
        _check(lib().sba_fwd(ctypes.byref(a)), "sba_fwd")
        if DEBUG_CHECK:
            check_status(ws, "sba_fwd")


def _launch_bwd(do, drem, q, k, v, carry, neg_log_acc, cu_seqlens, cu_has_leading_zero, max_seqlen, carry_slots, logit_scale,
                attend_current, add_remainder, dq, dk, dv):
    fixed = cu_seqlens is None
    with torch.cuda.device(q.device):
        a = _base_args(q, cu_seqlens, cu_has_leading_zero, max_seqlen, logit_scale, attend_current, carry_slots)
        a.add_remainder = 1 if add_remainder else 0
        a.row_stat = neg_log_acc.data_ptr() if neg_log_acc.numel() > 0 else None
        a.q, a.k, a.v, a.d_o, a.dq, a.dk, a.dv = (_tensor(t, fixed) for t in (q, k, v, do, dq, dk, dv))
        a.d_rem = _vector(drem, fixed)
        if carry.numel() > 0:
            a.carry = carry.data_ptr()
        else:
            a.recompute_carry = 1        # the forward kept no products: rebuild them in the backward's workspace
        nbytes = _workspace_bytes(a)[1]
        if BWD_WORKSPACE_LIMIT is not None and nbytes > BWD_WORKSPACE_LIMIT:
            # the smallest workspace the library accepts is the one of a single head
            heads, a.num_heads = a.num_heads, 1
            one_head = _workspace_bytes(a)[1]
            a.num_heads = heads
            nbytes = max(BWD_WORKSPACE_LIMIT, one_head)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
        a.workspace, a.workspace_bytes = ws.data_ptr(), nbytes
        if POISON:
            _poison(ws)
        if TRACE_EVENTS is not None:
            global LAST_BWD_KERNELS
            LAST_BWD_KERNELS = lib().sba_bwd_kernels(ctypes.byref(a))
        _check(lib().sba_bwd(ctypes.byref(a)), "sba_bwd")
        if DEBUG_CHECK:
            check_status(ws, "sba_bwd")


# The four launchers as out-parameter operators, registered for torch.compile the way the reference registers
# its own (sb_varlen_fwd.py:453, sb_varlen_bwd.py:541, sb_attn/sb_fwd.py:175, sb_attn/sb_bwd.py:207).  ``carry``
# replaces the reference's use of the saved ``neg_log_acc`` in the backward; an empty ``carry`` means "do not
# record it" in the forward and "rebuild it from q and k" in the backward.
@custom_op("varlen_fwd", mutates_args={"o", "rem", "neg_log_acc", "carry"})
def varlen_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens: torch.Tensor, cu_has_leading_zero: bool,
               max_seqlens: int, carry_slots: int, logit_scale: float, attend_current: bool, add_remainder: bool,
               o: torch.Tensor, rem: torch.Tensor, neg_log_acc: torch.Tensor, carry: torch.Tensor) -> None:
    _launch_fwd(q, k, v, cu_seqlens, cu_has_leading_zero, max_seqlens, carry_slots, logit_scale, attend_current, add_remainder,
                o, rem, neg_log_acc, carry)


@custom_op("varlen_bwd", mutates_args={"dq", "dk", "dv"})
def varlen_bwd(do: torch.Tensor, drem: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, carry: torch.Tensor,
               neg_log_acc: torch.Tensor, cu_seqlens: torch.Tensor, cu_has_leading_zero: bool, max_seqlens: int,
               carry_slots: int, logit_scale: float, attend_current: bool, add_remainder: bool, dq: torch.Tensor,
               dk: torch.Tensor, dv: torch.Tensor) -> None:
    _launch_bwd(do, drem, q, k, v, carry, neg_log_acc, cu_seqlens, cu_has_leading_zero, max_seqlens, carry_slots, logit_scale,
                attend_current, add_remainder, dq, dk, dv)


@custom_op("attn_fwd", mutates_args={"o", "rem", "neg_log_acc", "carry"})
def attn_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, logit_scale: float, attend_current: bool, add_remainder: bool,
             o: torch.Tensor, rem: torch.Tensor, neg_log_acc: torch.Tensor, carry: torch.Tensor) -> None:
    _launch_fwd(q, k, v, None, False, q.size(2), 0, logit_scale, attend_current, add_remainder, o, rem, neg_log_acc, carry)


@custom_op("attn_bwd", mutates_args={"dq", "dk", "dv"})
def attn_bwd(do: torch.Tensor, drem: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, carry: torch.Tensor,
             neg_log_acc: torch.Tensor, logit_scale: float, attend_current: bool, add_remainder: bool, dq: torch.Tensor,
             dk: torch.Tensor, dv: torch.Tensor) -> None:
    _launch_bwd(do, drem, q, k, v, carry, neg_log_acc, None, False, q.size(2), 0, logit_scale, attend_current, add_remainder,
                dq, dk, dv)


def _same_dtype(q, **others):
    for name, t in others.items():
        if t is not None and t.dtype != q.dtype:
            raise TypeError(f"{name} has dtype {t.dtype}, q has {q.dtype}: q, k, v and the gradients must share one dtype")


def forward(q, k, v, cu_seqlens, cu_has_leading_zero, max_seqlen, logit_scale, attend_current, want_carry, add_remainder=False,
            carry_slots=0):
    """Launch the forward.  Returns (o, rem, row_stat, carry or None).  Packed mode when cu_seqlens is given.
    ``carry`` is the buffer the backward needs; it is only produced when ``want_carry``.  With ``add_remainder`` the
    first output is ``o + rem[..., None] * v``.  ``carry_slots``: exact per-head size of ``carry`` from ``plan_host``
    (0 = the bound derived from ``max_seqlen``); the backward must be given the same value."""
    _require_gpu(q, k, v)
    fixed = cu_seqlens is None
    q, k, v = rows_contiguous(q), rows_contiguous(k), rows_contiguous(v)
    if q.dtype not in _DTYPES:
        raise TypeError(f"unsupported dtype {q.dtype}")
    _same_dtype(q, k=k, v=v)
    o = torch.empty_like(q)
    if o.stride(-1) != 1:
        o = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    rem = torch.empty(q.shape[:-1], dtype=q.dtype, device=q.device)
    row_stat = torch.empty(q.shape[:-1], dtype=torch.float32, device=q.device)
    n_carry = 0
    if want_carry:
        if fixed:
            n_carry = carry_elems(q.size(1), q.size(2), q.size(0), None, True)
        else:
            n_carry = carry_elems(q.size(0), q.size(1), cu_seqlens.numel() - (1 if cu_has_leading_zero else 0), max_seqlen, False,
                                  int(carry_slots))
    carry = torch.empty(n_carry, dtype=torch.float32, device=q.device)
    if fixed:
        attn_fwd(q, k, v, float(logit_scale), bool(attend_current), bool(add_remainder), o, rem, row_stat, carry)
    else:
        varlen_fwd(q, k, v, cu_seqlens, bool(cu_has_leading_zero), int(max_seqlen) if max_seqlen else 0, int(carry_slots),
                   float(logit_scale), bool(attend_current), bool(add_remainder), o, rem, row_stat, carry)
    return o, rem, row_stat, (carry if want_carry else None)


def backward(do, drem, q, k, v, carry, cu_seqlens, cu_has_leading_zero, max_seqlen, logit_scale, attend_current,
             row_stat=None, add_remainder=False, carry_slots=0):
    """Launch the backward.  Returns (dq, dk, dv).  ``row_stat`` (the forward's third output) is needed when the
    forward ran with ``add_remainder``.  Rows of a packed batch that belong to no sequence get zero gradients.
    ``carry=None``: the forward did not keep its products; the backward rebuilds them (16-bit dtypes only)."""
    _require_gpu(q, k, v, do, drem, carry)
    if carry is None:
        if q.dtype == torch.float32:
            raise TypeError("save_carry=False is not available for fp32 inputs")
        carry = torch.empty(0, dtype=torch.float32, device=q.device)
    fixed = cu_seqlens is None
    _same_dtype(q, k=k, v=v, do=do)
    do = rows_contiguous(do)
    q, k, v = rows_contiguous(q), rows_contiguous(k), rows_contiguous(v)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    if drem is None:
        drem = torch.zeros(q.shape[:-1], dtype=q.dtype, device=q.device)
    elif drem.dtype != q.dtype:
        drem = drem.to(q.dtype)
    if add_remainder and row_stat is None:
        raise ValueError("the backward of add_remainder needs the forward's row_stat")
    if row_stat is None:
        row_stat = torch.empty(0, dtype=torch.float32, device=q.device)
    if fixed:
        attn_bwd(do, drem, q, k, v, carry, row_stat, float(logit_scale), bool(attend_current), bool(add_remainder), dq, dk, dv)
    else:
        varlen_bwd(do, drem, q, k, v, carry, row_stat, cu_seqlens, bool(cu_has_leading_zero),
                   int(max_seqlen) if max_seqlen else 0, int(carry_slots), float(logit_scale), bool(attend_current),
                   bool(add_remainder), dq, dk, dv)
    return dq, dk, dv
