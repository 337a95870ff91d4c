"""Tensor-level wrappers over the katz_hip C ABI.

Every function validates shapes / dtypes / device, passes raw device pointers and torch's current
HIP stream to the library, and returns torch tensors.  Work is enqueued on the current stream, so the
calls compose with other torch ops and with torch.cuda.graph capture.  Nothing here computes on the
CPU: without a GPU (or without the built library) the functions raise.
"""
from __future__ import annotations

import contextlib
import ctypes
import math
import os
import weakref
from typing import Optional, Sequence

import torch

from . import _lib

BF16 = torch.bfloat16

# When set to a list, lora_linear / attention append their problem sizes to it (benchmark accounting).
CALL_LOG = None


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _req(t: torch.Tensor, dtype, name: str) -> None:
    if not t.is_cuda:
        raise _lib.KatzHipError(f"{name} must live on the GPU (got {t.device}); katz_hip has no CPU path")
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


# --------------------------------------------------------------------------------------- K1
# Weight prefetch: a linear / convolution launch can touch the operands of the launch that follows it (weights, and the
# packed adapter matrices), so that those wait in the memory-side cache (kh_set_weight_prefetch).  Which operands follow
# which is learned from the previous pass over the SAME model: hints are learned and issued only inside
# `weight_prefetch_scope(model)`, which the UNet / ControlNet forward opens around its body.  Every model has a table of
# its own and a scope starts with no predecessor, so a pair (launch, next launch) never spans two models or two
# forwards: a captured graph of a model therefore holds hinted pointers to that model's own tensors only, which it needs
# alive anyway.  Launches outside any scope (a layer or an op called on its own) neither learn nor hint.
# The tables hold weak references only: a hint never keeps a tensor alive, and a dead one is dropped instead of hinted.
WEIGHT_PREFETCH = os.getenv("KATZ_WEIGHT_PREFETCH", "1") != "0"
PREFETCH_MIN_K = int(os.getenv("KATZ_PREFETCH_MIN_K", "2560"))
PREFETCH_SMALL_BYTES = int(os.getenv("KATZ_PREFETCH_SMALL_BYTES", str(4 << 20)))
_pf_tables: "weakref.WeakKeyDictionary" = weakref.WeakKeyDictionary()   # model -> its table (below)
_pf_next: list = [None]  # table of the running scope: data_ptr of a launch's weights -> weak refs to (weights, a_cat, b_cat) of the launch after it
_pf_last: list = [None]
_pf_shrink_a: list = [None]   # A_cat of a separate shrink launch, for the hint of the GEMM it belongs to


@contextlib.contextmanager
def weight_prefetch_scope(owner):
    """One forward of one model: launches inside learn from / hint at `owner`'s own table, starting without a predecessor;
    on exit the enclosing scope (normally none) is restored and whatever hint is still pending in the library is dropped."""
    table = _pf_tables.get(owner)
    if table is None:
        table = _pf_tables[owner] = {}
    saved = (_pf_next[0], _pf_last[0], _pf_shrink_a[0])
    _pf_next[0], _pf_last[0], _pf_shrink_a[0] = table, None, None
    try:
        yield table
    finally:
        _pf_next[0], _pf_last[0], _pf_shrink_a[0] = saved
        if WEIGHT_PREFETCH and _lib.is_loaded():
            _lib.load().kh_set_weight_prefetch(None, 0)


def _weight_prefetch_hint(weight: torch.Tensor, a_cat: Optional[torch.Tensor] = None,
                          b_cat: Optional[torch.Tensor] = None) -> None:
    if not WEIGHT_PREFETCH:
        return
    lib = _lib.load()
    # whatever an earlier call left pending (its launch was refused before it took the hint) must not reach this launch
    lib.kh_set_weight_prefetch(None, 0)
    table = _pf_next[0]
    if a_cat is None and _pf_shrink_a[0] is not None:
        a_cat = _pf_shrink_a[0]()
    _pf_shrink_a[0] = None
    if table is None:
        return
    key = weight.data_ptr()
    last = _pf_last[0]
    if last is not None and last != key:
        table[last] = tuple(None if t is None else weakref.ref(t) for t in (weight, a_cat, b_cat))
        if len(table) > 65536:     # weights come and go: forget everything rather than grow without bound
            table.clear()
    _pf_last[0] = key
    nxt = table.get(key)
    if nxt is None:
        return
    live = [None if r is None else r() for r in nxt]
    w_next = live[0]
    if w_next is None:                # the tensor that followed last time is gone
        del table[key]
        return
    # The prefetch is not free for the launch that carries it (its own first operands queue behind it: up to 3.5 us
    # for 26 MB), so weights are only hinted where meeting them in HBM costs more than that: long rows (K >= 2560,
    # the feed-forward output projections and the 3x3 convolutions), whose launches are latency-bound on their
    # operand stream -- and small ones (<= 4 MB: the d x d layers), which delay their carrier by well under a microsecond
    # (measured: 24.19 -> 23.80 ms per step with them, 24.4 with every weight hinted).  The adapter matrices are small
    # and always hinted.
    k_next = w_next.shape[-1] * (9 if w_next.dim() == 4 else 1)
    small = w_next.numel() * w_next.element_size() <= PREFETCH_SMALL_BYTES
    for t in ((w_next if (k_next >= PREFETCH_MIN_K or small) else None),) + tuple(live[1:]):
        if t is not None:
            lib.kh_set_weight_prefetch(t.data_ptr(), t.numel() * t.element_size())


def lora_linear(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    a_cat: Optional[torch.Tensor] = None,
    b_cat: Optional[torch.Tensor] = None,
    col_scale: Optional[torch.Tensor] = None,
    residual: Optional[torch.Tensor] = None,
    geglu: bool = False,
    tile: int = 0,
    out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """y = x W^T + b + ((x A_cat^T) * col_scale) B_cat^T (+ residual); bf16 or fp32 by x.dtype.

    a_cat [R,K], b_cat [N,R], col_scale [R] fp32 describe the active adapters concatenated along the
    rank axis (R % 32 == 0 for bf16).  With geglu=True the rows of weight / bias / b_cat must be in the
    interleaved (32 value, 32 gate) order produced by `katz_amd.lora.interleave_geglu_rows`.
    """
    lib = _lib.load()
    K = x.shape[-1]
    N = weight.shape[0]
    M = x.numel() // K
    dt = x.dtype
    _req(x, dt, "x"); _req(weight, dt, "weight")
    if weight.shape[1] != K:
        raise ValueError(f"weight {tuple(weight.shape)} does not match x[..., {K}]")
    R = 0
    if a_cat is not None:
        _req(a_cat, dt, "a_cat"); _req(b_cat, dt, "b_cat"); _req(col_scale, torch.float32, "col_scale")
        R = a_cat.shape[0]
        if a_cat.shape != (R, K) or b_cat.shape != (N, R) or col_scale.shape != (R,):
            raise ValueError("a_cat/b_cat/col_scale shapes must be [R,K], [N,R], [R]")
    if bias is not None:
        _req(bias, dt, "bias")
    n_out = N // 2 if geglu else N
    out_shape = tuple(x.shape[:-1]) + (n_out,)
    if residual is not None:
        _req(residual, dt, "residual")
        if residual.numel() != M * N:
            raise ValueError("residual must have the shape of the output")
    if out is None:
        out = torch.empty(out_shape, dtype=dt, device=x.device)
    else:
        _req(out, dt, "out")
        if out.numel() != M * n_out:
            raise ValueError("out has the wrong size")
    if CALL_LOG is not None:
        CALL_LOG.append(("lora_linear", M, N, K, R, bool(geglu), residual is not None))
    if dt == BF16:
        flags = (1 if geglu else 0) | ((tile & 0xFF) << 8)
        _weight_prefetch_hint(weight, a_cat, b_cat)
        rc = lib.kh_lora_linear_bf16(_ptr(x), _ptr(weight), _ptr(bias), _ptr(a_cat), _ptr(b_cat), _ptr(col_scale),
                                     _ptr(residual), _ptr(out), M, N, K, R, flags, _stream())
    elif dt == torch.float32:
        if geglu:
            raise ValueError("the GEGLU epilogue exists for bf16 only")
        rc = lib.kh_lora_linear_f32(_ptr(x), _ptr(weight), _ptr(bias), _ptr(a_cat), _ptr(b_cat), _ptr(col_scale),
                                    _ptr(residual), _ptr(out), M, N, K, R, _stream())
    else:
        raise TypeError(f"lora_linear supports bfloat16 and float32, got {dt}")
    _lib.check(rc, "kh_lora_linear")
    return out


def lora_shrink(x: torch.Tensor, a_cat: torch.Tensor, col_scale: torch.Tensor, out: Optional[torch.Tensor] = None):
    """t = bf16((x A_cat^T) * col_scale), [M, R]; A_cat may stack the adapters of several layers that read x."""
    lib = _lib.load()
    _req(x, BF16, "x"); _req(a_cat, BF16, "a_cat"); _req(col_scale, torch.float32, "col_scale")
    K = x.shape[-1]
    M = x.numel() // K
    R = a_cat.shape[0]
    if a_cat.shape != (R, K) or col_scale.shape != (R,):
        raise ValueError("a_cat / col_scale must be [R,K] / [R]")
    if out is None:
        out = torch.empty((M, R), dtype=BF16, device=x.device)
    if CALL_LOG is not None:
        CALL_LOG.append(("lora_shrink", M, K, R))
    _pf_shrink_a[0] = weakref.ref(a_cat)
    rc = lib.kh_lora_shrink_bf16(_ptr(x), _ptr(a_cat), _ptr(col_scale), _ptr(out), M, K, R, _stream())
    _lib.check(rc, "kh_lora_shrink_bf16")
    return out


def _no_coop_bit() -> int:
    """Flag bit 24 of the split / norm entry points: inside side_branch() the cooperative in-launch shrink is off.  Its
    workgroups wait for each other, and two such launches running side by side on two streams could each hold the CUs
    the other one's last workgroups need."""
    return (1 << 24) if _ws_slot[0] > 0 else 0


def _r_used_bits(r_used: int, R: int) -> int:
    if r_used < 0 or r_used > R or r_used % 16:
        raise ValueError(f"r_used must be a multiple of 16 in [0, {R}], got {r_used}")
    return r_used // 16


def lora_linear_pre(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], t: torch.Tensor,
                    b_cat: torch.Tensor, residual: Optional[torch.Tensor] = None, geglu: bool = False,
                    tile: int = 0, n_split: int = 0, r_used: int = 0) -> torch.Tensor:
    """y = x W^T + b + t B_cat^T (+ residual | GEGLU) with t = lora_shrink(x, ...)[:, cols] (a column
    slice of a wider shrink result is fine: only its last axis must be contiguous).  n_split > 0: weight /
    bias / b_cat stack several layers of n_split rows each and t holds their shrink results side by side.
    r_used > 0 (a multiple of 16): rank columns >= r_used of t and b_cat are all zero (padding)."""
    lib = _lib.load()
    _req(x, BF16, "x"); _req(weight, BF16, "weight"); _req(b_cat, BF16, "b_cat")
    K = x.shape[-1]
    N = weight.shape[0]
    M = x.numel() // K
    R = b_cat.shape[1]
    t_cols = R * (N // n_split) if n_split else R
    if t.dtype != BF16 or not t.is_cuda or t.dim() != 2 or t.stride(1) != 1 or t.shape != (M, t_cols):
        raise ValueError(f"t must be a bfloat16 [M,{t_cols}] GPU matrix with a contiguous last axis")
    if weight.shape[1] != K or b_cat.shape[0] != N:
        raise ValueError("weight / b_cat do not match x")
    if bias is not None:
        _req(bias, BF16, "bias")
    if residual is not None:
        _req(residual, BF16, "residual")
        if residual.numel() != M * N:
            raise ValueError("residual must have the shape of the output")
    n_out = N // 2 if geglu else N
    out = torch.empty(tuple(x.shape[:-1]) + (n_out,), dtype=BF16, device=x.device)
    if CALL_LOG is not None:
        CALL_LOG.append(("lora_linear", M, N, K, R, bool(geglu), residual is not None))
    flags = (1 if geglu else 0) | ((tile & 0xFF) << 8) | (_r_used_bits(r_used, R) << 16)
    _weight_prefetch_hint(weight, None, b_cat)
    rc = lib.kh_lora_linear_pre_bf16(_ptr(x), _ptr(weight), _ptr(bias), _ptr(t), t.stride(0), n_split, _ptr(b_cat),
                                     _ptr(residual), _ptr(out), M, N, K, R, flags, _stream())
    _lib.check(rc, "kh_lora_linear_pre_bf16")
    return out


# Counters of kh_lora_linear_split_bf16's in-launch shrink.  Every call needs ceil(M / 128) + 1 zeroed int32 and leaves
# them dirty, so they come from one arena per device: calls take consecutive slices, and `split_counters_reset`
# clears the WHOLE arena with one fill kernel (256 KB: as cheap as any fill) and starts over.  The whole arena, not
# just what the host handed out since the last reset: a reset recorded into a HIP graph runs at replay time, when the
# host's count says nothing about what eager forwards or other graphs have dirtied in between.  The UNet / ControlNet
# forward resets at its start (inside a captured graph that is one fill node per step and the same slices on every
# replay); a caller that never resets is served until the arena is full, then it is reset for him.  One stream per
# device: a reset must not overtake launches that still use their slices (two models side by side on two streams:
# clear once before the fork and run both under `split_counters_held`).
SPLIT_ARENA_INTS = 1 << 16
_split_arena: dict = {}     # (device type, index) -> [buffer, ints handed out, last slice, ever used]


def _arena(device):
    key = (device.type, device.index)
    st = _split_arena.get(key)
    if st is None:
        if torch.cuda.is_current_stream_capturing():
            # memory allocated during a capture belongs to the graph's pool and dies with the graph
            raise RuntimeError("katz_amd: run the step once eagerly before capturing it (the LoRA counter arena is "
                               "allocated on first use and must outlive the graph)")
        st = [torch.zeros(SPLIT_ARENA_INTS, dtype=torch.int32, device=device), 0, None, False]
        _split_arena[key] = st
    return st


_arena_held: list = [0]


@contextlib.contextmanager
def split_counters_held():
    """Inside this context `split_counters_reset` does nothing: for a caller that runs two models side by side on two
    streams (a ControlNet beside the UNet's down blocks), clears the arena ONCE before the fork and must not have one
    model's reset wipe or re-issue the slices the other's launches are using."""
    _arena_held[0] += 1
    try:
        yield
    finally:
        _arena_held[0] -= 1


def split_counters_reset(device) -> None:
    """Clear every counter of the device's arena with one fill kernel.  Outside graph capture the fill is skipped
    while no counter has ever been handed out; under capture it is always recorded, because by the time the graph is
    replayed other forwards may have dirtied the arena."""
    if _arena_held[0]:
        return
    st = _arena(device)
    if st[3] or torch.cuda.is_current_stream_capturing():
        st[0].zero_()
    st[1] = 0


class SplitTimeoutError(_lib.KatzHipError):
    """A bounded wait inside kh_lora_linear_split_bf16 ran out: results since the last check are not trustworthy."""


def split_timeouts(device=None, clear: bool = False) -> int:
    """How many in-launch waits of lora_linear_split have run out on `device` since the last clearing call.
    Synchronises with the device."""
    import ctypes

    lib = _lib.load()
    n = ctypes.c_int32(0)
    with torch.cuda.device(device if device is not None else torch.cuda.current_device()):
        rc = lib.kh_lora_split_timeouts(ctypes.byref(n), 1 if clear else 0)
    _lib.check(rc, "kh_lora_split_timeouts")
    return int(n.value)


def check_split_timeouts(device=None) -> None:
    """Raise SplitTimeoutError if any in-launch wait has run out since the last check (and clear the count).  Call it
    where the host synchronises anyway: after a denoise loop, after a benchmark's timed region, in tests."""
    n = split_timeouts(device, clear=True)
    if n:
        raise SplitTimeoutError(f"{n} in-launch shrink wait(s) of kh_lora_linear_split_bf16 timed out on {device}: "
                                "the LoRA linears of the affected steps read an incomplete shrink result")


def _split_counters(device, M: int) -> torch.Tensor:
    return _arena_ints(device, (M + 127) // 128 + 1)   # KH_SPLIT_COUNTER_INTS(M)


def _arena_ints(device, n: int) -> torch.Tensor:
    """n zeroed int32 of the device's counter arena (zero since the last split_counters_reset)."""
    st = _arena(device)
    if st[1] + n > SPLIT_ARENA_INTS:
        if _arena_held[0]:
            raise RuntimeError("katz_amd: the LoRA counter arena is full inside split_counters_held()")
        split_counters_reset(device)
    st[2] = st[0][st[1]:st[1] + n]
    st[1] += n
    st[3] = True
    return st[2]


def split_counters_last(device) -> Optional[torch.Tensor]:
    """The counters of the most recent lora_linear_split call on this device (for tests: arrivals per row block, then
    the time-out flag)."""
    return _arena(device)[2]


def lora_linear_split(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], a_cat: torch.Tensor,
                      col_scale: torch.Tensor, b_cat: torch.Tensor, residual: Optional[torch.Tensor] = None,
                      geglu: bool = False, two_launches: bool = False, n_split: int = 0, r_used: int = 0) -> torch.Tensor:
    """y = x W^T + b + ((x A_cat^T) * col_scale) B_cat^T (+ residual | GEGLU): shrink, base GEMM and expand, with
    the shrink inside the GEMM launch where that pays (see kh_lora_linear_split_bf16).  n_split > 0: weight / bias /
    b_cat stack several layers of n_split rows each and a_cat / col_scale stack their A matrices."""
    lib = _lib.load()
    _req(x, BF16, "x"); _req(weight, BF16, "weight"); _req(a_cat, BF16, "a_cat"); _req(b_cat, BF16, "b_cat")
    _req(col_scale, torch.float32, "col_scale")
    K = x.shape[-1]
    N = weight.shape[0]
    M = x.numel() // K
    RT = a_cat.shape[0]
    R = b_cat.shape[1]
    if n_split and (N % n_split or RT != (N // n_split) * R):
        raise ValueError("stacked layers: a_cat must have N / n_split * R rows")
    if not n_split and RT != R:
        raise ValueError("a_cat and b_cat disagree on the rank")
    if weight.shape[1] != K or a_cat.shape != (RT, K) or b_cat.shape != (N, R) or col_scale.shape != (RT,):
        raise ValueError("weight / a_cat / b_cat / col_scale do not match x")
    if bias is not None:
        _req(bias, BF16, "bias")
    if residual is not None:
        _req(residual, BF16, "residual")
        if residual.numel() != M * N:
            raise ValueError("residual must have the shape of the output")
    n_out = N // 2 if geglu else N
    out = torch.empty(tuple(x.shape[:-1]) + (n_out,), dtype=BF16, device=x.device)
    t = torch.empty((M, RT), dtype=BF16, device=x.device)
    cnt = _split_counters(x.device, M)
    flags = (1 if geglu else 0) | ((1 if two_launches else 0) << 8) | (_r_used_bits(r_used, R) << 16) | _no_coop_bit()
    if CALL_LOG is not None:   # one entry per kernel launch
        if lib.kh_lora_linear_split_launches(M, N, K, R, n_split, flags) == 2:
            CALL_LOG.append(("lora_shrink", M, K, RT))
        CALL_LOG.append(("lora_linear", M, N, K, R, bool(geglu), residual is not None))
    _weight_prefetch_hint(weight, a_cat, b_cat)
    rc = lib.kh_lora_linear_split_bf16(_ptr(x), _ptr(weight), _ptr(bias), _ptr(a_cat), _ptr(col_scale), _ptr(b_cat), _ptr(t),
                                       _ptr(cnt), _ptr(residual), _ptr(out), M, N, K, R, n_split, flags, _stream())
    _lib.check(rc, "kh_lora_linear_split_bf16")
    return out


LN_SLOTS = 16   # KH_LN_SLOTS: (sum, sum of squares) pairs per row in a row-statistics buffer


def row_stats_buffer(M: int, device) -> torch.Tensor:
    """float32 [16, M, 2]: what a linear with stats_out= writes and a linear with ln= reads (kh_lora_linear_norm_bf16)."""
    return torch.empty((LN_SLOTS, M, 2), dtype=torch.float32, device=device)


def lora_linear_norm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                     a_cat: Optional[torch.Tensor] = None, col_scale: Optional[torch.Tensor] = None,
                     b_cat: Optional[torch.Tensor] = None, residual: Optional[torch.Tensor] = None, geglu: bool = False,
                     two_launches: bool = False, n_split: int = 0, r_used: int = 0, ln=None,
                     stats_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The LoRA linear with a LayerNorm folded in front of it and / or the row statistics for one behind it
    (kh_lora_linear_norm_bf16).

    ln = (part, c1, c2, ca1, ca2, eps): x is then the UN-normalised input, `part` the statistics of its rows (written by
    the linear that produced x), weight / a_cat already carry the norm's weight, c1 / c2 (float [N]) and ca1 / ca2 (float
    [rows of a_cat], None without adapters) are the folded terms; bias must be None (it is part of c2).
    stats_out: a row_stats_buffer for the rows of the result (after bias and residual)."""
    lib = _lib.load()
    _req(x, BF16, "x"); _req(weight, BF16, "weight")
    K = x.shape[-1]
    N = weight.shape[0]
    M = x.numel() // K
    R = RT = 0
    if a_cat is not None:
        _req(a_cat, BF16, "a_cat"); _req(b_cat, BF16, "b_cat"); _req(col_scale, torch.float32, "col_scale")
        RT, R = a_cat.shape[0], b_cat.shape[1]
        if n_split and (N % n_split or RT != (N // n_split) * R):
            raise ValueError("stacked layers: a_cat must have N / n_split * R rows")
        if not n_split and RT != R:
            raise ValueError("a_cat and b_cat disagree on the rank")
        if a_cat.shape != (RT, K) or b_cat.shape != (N, R) or col_scale.shape != (RT,):
            raise ValueError("a_cat / b_cat / col_scale do not match x and weight")
    if weight.shape[1] != K:
        raise ValueError("weight does not match x")
    if bias is not None:
        _req(bias, BF16, "bias")
    if residual is not None:
        _req(residual, BF16, "residual")
        if residual.numel() != M * N:
            raise ValueError("residual must have the shape of the output")
    part = c1 = c2 = ca1 = ca2 = None
    eps = 0.0
    if ln is not None:
        part, c1, c2, ca1, ca2, eps = ln
        if bias is not None:
            raise ValueError("with a folded LayerNorm the bias belongs into c2")
        for t_, n_, name in ((c1, N, "c1"), (c2, N, "c2")) + (((ca1, RT, "ca1"), (ca2, RT, "ca2")) if R else ()):
            _req(t_, torch.float32, name)
            if t_.numel() != n_:
                raise ValueError(f"{name} must have {n_} elements")
        _req(part, torch.float32, "ln part")
        if part.numel() != M * LN_SLOTS * 2:
            raise ValueError("ln part must be a row_stats_buffer for the rows of x")
    if stats_out is not None:
        _req(stats_out, torch.float32, "stats_out")
        if stats_out.numel() != M * LN_SLOTS * 2:
            raise ValueError("stats_out must be a row_stats_buffer for the rows of the output")
    n_out = N // 2 if geglu else N
    out = torch.empty(tuple(x.shape[:-1]) + (n_out,), dtype=BF16, device=x.device)
    t = cnt = None
    if R:
        t = torch.empty((M, RT), dtype=BF16, device=x.device)
        cnt = _split_counters(x.device, M)
    flags = (1 if geglu else 0) | ((1 if two_launches else 0) << 8) | (_r_used_bits(r_used, R) << 16 if R else 0) | _no_coop_bit()
    if CALL_LOG is not None:   # one entry per kernel launch
        if R and lib.kh_lora_linear_split_launches(M, N, K, R, n_split, flags) == 2:
            CALL_LOG.append(("lora_shrink", M, K, RT))
        CALL_LOG.append(("lora_linear", M, N, K, R, bool(geglu), residual is not None, ln is not None, stats_out is not None))
    _weight_prefetch_hint(weight, a_cat, b_cat)
    rc = lib.kh_lora_linear_norm_bf16(_ptr(x), _ptr(weight), _ptr(bias), _ptr(a_cat), _ptr(col_scale), _ptr(b_cat), _ptr(t),
                                      _ptr(cnt), _ptr(residual), _ptr(out), _ptr(part), _ptr(c1), _ptr(c2), _ptr(ca1), _ptr(ca2),
                                      float(eps), _ptr(stats_out), M, N, K, R, n_split, flags, _stream())
    _lib.check(rc, "kh_lora_linear_norm_bf16")
    return out


def lora_linear_xattn_ok(M: int, N: int, K: int, R: int, T: int, S: int, heads: int) -> bool:
    """Does lora_linear_xattn take this query projection ([M,K] -> [M,N], adapters' padded rank R) and attention (T queries
    and S keys per sample, 64-wide heads)?"""
    return N == heads * 64 and bool(_lib.load().kh_lora_linear_xattn_ok(M, N, K, R, T, S))


def lora_linear_xattn(x: torch.Tensor, weight: torch.Tensor, k: torch.Tensor, v: torch.Tensor, heads: int,
                      scale: Optional[float] = None, bias: Optional[torch.Tensor] = None,
                      a_cat: Optional[torch.Tensor] = None, col_scale: Optional[torch.Tensor] = None,
                      b_cat: Optional[torch.Tensor] = None, two_launches: bool = False, r_used: int = 0,
                      ln=None) -> torch.Tensor:
    """attention(lora_linear_norm(x, weight, ...), k, v) in one launch (kh_lora_linear_xattn_bf16): the query projection of a
    cross-attention over a short context (S <= 96) whose 128 x 128 output tiles (128 queries of two heads) go through the
    attention inside the GEMM's epilogue instead of to memory.  x [B,T,K]; k / v [B,S,heads*64] (last-dim-contiguous
    views); the other arguments as for lora_linear_norm.  Returns [B,T,heads*64]."""
    lib = _lib.load()
    _req(x, BF16, "x"); _req(weight, BF16, "weight")
    if x.dim() != 3:
        raise ValueError("x must be [B,T,K]")
    B, T, K = x.shape
    N = weight.shape[0]
    M = B * T
    S = k.shape[1]
    if weight.shape[1] != K or N != heads * 64:
        raise ValueError("weight must be [heads*64, K]")
    for n, t in (("k", k), ("v", v)):
        if not t.is_cuda or t.dtype != BF16 or t.stride(-1) != 1 or t.shape != (B, S, N):
            raise ValueError(f"{n} must be a bfloat16 [B,S,heads*64] GPU tensor with a contiguous last axis")
    R = 0
    if a_cat is not None:
        _req(a_cat, BF16, "a_cat"); _req(b_cat, BF16, "b_cat"); _req(col_scale, torch.float32, "col_scale")
        R = b_cat.shape[1]
        if a_cat.shape != (R, K) or b_cat.shape != (N, R) or col_scale.shape != (R,):
            raise ValueError("a_cat / b_cat / col_scale do not match x and weight")
    if bias is not None:
        _req(bias, BF16, "bias")
    part = c1 = c2 = ca1 = ca2 = None
    eps = 0.0
    if ln is not None:
        part, c1, c2, ca1, ca2, eps = ln
        if bias is not None:
            raise ValueError("with a folded LayerNorm the bias belongs into c2")
        for t_, n_, name in ((c1, N, "c1"), (c2, N, "c2")) + (((ca1, R, "ca1"), (ca2, R, "ca2")) if R else ()):
            _req(t_, torch.float32, name)
            if t_.numel() != n_:
                raise ValueError(f"{name} must have {n_} elements")
        _req(part, torch.float32, "ln part")
        if part.numel() != M * LN_SLOTS * 2:
            raise ValueError("ln part must be a row_stats_buffer for the rows of x")
    if scale is None:
        scale = 1.0 / 8.0
    out = torch.empty((B, T, N), dtype=BF16, device=x.device)
    t = cnt = None
    if R:
        t = torch.empty((M, R), dtype=BF16, device=x.device)
        cnt = _split_counters(x.device, M)
    # bit 24: the cooperative shrink belongs to another kernel family (the launch count below must not count on it)
    flags = ((1 if two_launches else 0) << 8) | (_r_used_bits(r_used, R) << 16 if R else 0) | (1 << 24)
    if CALL_LOG is not None:   # one entry per kernel launch
        if R and lib.kh_lora_linear_split_launches(M, N, K, R, 0, flags) == 2:
            CALL_LOG.append(("lora_shrink", M, K, R))
        CALL_LOG.append(("lora_linear_xattn", M, N, K, R, heads, T, S))
    _weight_prefetch_hint(weight, a_cat, b_cat)
    rc = lib.kh_lora_linear_xattn_bf16(_ptr(x), _ptr(weight), _ptr(bias), _ptr(a_cat), _ptr(col_scale), _ptr(b_cat), _ptr(t),
                                       _ptr(cnt), _ptr(part), _ptr(c1), _ptr(c2), _ptr(ca1), _ptr(ca2), float(eps),
                                       _ptr(k), _ptr(v), _ptr(out), M, N, K, R, T, S, k.stride(1), v.stride(1), out.stride(1),
                                       k.stride(0), v.stride(0), float(scale), flags, _stream())
    _lib.check(rc, "kh_lora_linear_xattn_bf16")
    return out


def lora_merge_grouped(weights: Sequence[torch.Tensor], ups: Sequence[torch.Tensor], downs: Sequence[torch.Tensor],
                       scale: float = 1.0, layer_scales: Optional[Sequence[float]] = None) -> None:
    """W_l += scale * layer_scales[l] * up_l @ down_l for all layers in ONE launch, in place (kh_lora_merge_grouped_bf16).
    weights: contiguous bf16 [N,K] GPU tensors, each at most once; ups [N,r] / downs [r,K]: contiguous GPU tensors, all
    bfloat16 or all float16, r <= 128.  Tensors derived from a weight notice the change through its version counter,
    which is bumped here as an in-place torch op would."""
    lib = _lib.load()
    n = len(weights)
    if n == 0:
        return
    if len(ups) != n or len(downs) != n or (layer_scales is not None and len(layer_scales) != n):
        raise ValueError("weights, ups, downs (and layer_scales) must have one entry per layer")
    dev = weights[0].device
    op_dtype = ups[0].dtype
    if op_dtype not in (BF16, torch.float16):
        raise TypeError("adapter matrices must be bfloat16 or float16")
    rows, starts, max_rank, seen = [], [0], 0, set()
    for w, u, d in zip(weights, ups, downs):
        if not w.is_cuda or w.dtype != BF16 or w.dim() != 2 or not w.is_contiguous() or w.device != dev:
            raise ValueError("every weight must be a contiguous 2-D bfloat16 tensor on one GPU")
        N, K = w.shape
        r = d.shape[0]
        for t, shape, name in ((u, (N, r), "up"), (d, (r, K), "down")):
            if not t.is_cuda or t.device != dev or t.dtype != op_dtype or not t.is_contiguous() or tuple(t.shape) != shape:
                raise ValueError(f"{name} must be a contiguous {op_dtype} {shape} tensor on {dev}, got {t.dtype} {tuple(t.shape)}")
        if r < 1 or r > 128:
            raise ValueError(f"rank {r} outside 1..128")
        if w.data_ptr() in seen:
            raise ValueError("a weight appears twice in one merge (the tiles of the two rows would race)")
        seen.add(w.data_ptr())
        rows.append((w.data_ptr(), u.data_ptr(), d.data_ptr(), N, K, r))
        starts.append(starts[-1] + ((N + 127) // 128) * ((K + 127) // 128))
        max_rank = max(max_rank, r)
    table = torch.tensor(rows, dtype=torch.int64).to(dev, non_blocking=True)
    tile_start = torch.tensor(starts, dtype=torch.int32).to(dev, non_blocking=True)
    ls = None if layer_scales is None else torch.tensor(list(layer_scales), dtype=torch.float32).to(dev, non_blocking=True)
    rc = lib.kh_lora_merge_grouped_bf16(_ptr(table), _ptr(tile_start), _ptr(ls), n, starts[-1], max_rank, float(scale),
                                        1 if op_dtype == torch.float16 else 0, _stream())
    _lib.check(rc, "kh_lora_merge_grouped_bf16")
    for w in weights:
        torch.autograd.graph.increment_version(w)
    # the table tensors are freed when this returns: torch's caching allocator keeps the memory valid for work already
    # enqueued on the current stream, which is where the kernel runs


def lora_linear_grouped(x: torch.Tensor, table: torch.Tensor, M: int, N: int, K: int, R: int, ldt: int) -> None:
    """y_g = x W_g^T + b_g + t_g B_cat_g^T for every row {W, bias, B_cat, t, y} of the int64 device
    `table` [n_groups, 5] in one launch; the caller owns every buffer the table points to."""
    lib = _lib.load()
    _req(x, BF16, "x"); _req(table, torch.int64, "table")
    if table.dim() != 2 or table.shape[1] != 5:
        raise ValueError("table must be [n_groups, 5] int64")
    if x.numel() != M * K:
        raise ValueError("x does not match M x K")
    if CALL_LOG is not None:
        CALL_LOG.append(("lora_linear_grouped", M, N, K, R, int(table.shape[0])))
    rc = lib.kh_lora_linear_grouped_bf16(_ptr(x), _ptr(table), table.shape[0], ldt, M, N, K, R, 0, _stream())
    _lib.check(rc, "kh_lora_linear_grouped_bf16")


# --------------------------------------------------------------------------------------- K2
def sgmv_shrink(x, a_all, seg_start, seg_adapter, adapter_rank, max_seg_rows: int, out=None):
    """t[rows, :r_a] = x[rows] A_a^T per segment. a_all [n_adapters, RP, K]; returns t [rows, RP]."""
    lib = _lib.load()
    _req(x, BF16, "x"); _req(a_all, BF16, "a_all")
    for n, t in (("seg_start", seg_start), ("seg_adapter", seg_adapter), ("adapter_rank", adapter_rank)):
        _req(t, torch.int32, n)
    rows, K = x.shape
    RP = a_all.shape[1]
    if a_all.shape[2] != K:
        raise ValueError("a_all must be [n_adapters, RP, K]")
    if out is None:
        out = torch.zeros((rows, RP), dtype=BF16, device=x.device)
    nseg = seg_adapter.numel()
    rc = lib.kh_sgmv_shrink_bf16(_ptr(x), _ptr(a_all), _ptr(out), _ptr(seg_start), _ptr(seg_adapter),
                                 _ptr(adapter_rank), nseg, max_seg_rows, K, RP, _stream())
    _lib.check(rc, "kh_sgmv_shrink_bf16")
    return out


def sgmv_expand_(y, t, b_all, seg_start, seg_adapter, adapter_rank, adapter_scale, max_seg_rows: int):
    """y[rows] += scale_a * t[rows, :r_a] B_a^T per segment, in place. b_all [n_adapters, N, RP]."""
    lib = _lib.load()
    _req(y, BF16, "y"); _req(t, BF16, "t"); _req(b_all, BF16, "b_all"); _req(adapter_scale, torch.float32, "adapter_scale")
    rows, N = y.shape
    RP = b_all.shape[2]
    if b_all.shape[1] != N or t.shape != (rows, RP):
        raise ValueError("b_all must be [n_adapters, N, RP] and t [rows, RP]")
    nseg = seg_adapter.numel()
    rc = lib.kh_sgmv_expand_bf16(_ptr(t), _ptr(b_all), _ptr(y), _ptr(seg_start), _ptr(seg_adapter),
                                 _ptr(adapter_rank), _ptr(adapter_scale), nseg, max_seg_rows, N, RP, _stream())
    _lib.check(rc, "kh_sgmv_expand_bf16")
    return y


def sgmv_fused_(y, x, a_all, b_all, seg_start, seg_adapter, adapter_rank, adapter_scale, max_seg_rows: int):
    """y[rows] += scale_a * bf16(x[rows] A_a^T) B_a^T per segment, in place, in ONE launch (kh_sgmv_fused_bf16): the
    arithmetic of sgmv_shrink followed by sgmv_expand_ without the round trip of t.  K % 64 == 0, N % 128 == 0."""
    lib = _lib.load()
    _req(y, BF16, "y"); _req(x, BF16, "x"); _req(a_all, BF16, "a_all"); _req(b_all, BF16, "b_all")
    _req(adapter_scale, torch.float32, "adapter_scale")
    for n, t in (("seg_start", seg_start), ("seg_adapter", seg_adapter), ("adapter_rank", adapter_rank)):
        _req(t, torch.int32, n)
    rows, K = x.shape
    N = y.shape[1]
    RP = a_all.shape[1]
    if y.shape[0] != rows or a_all.shape[2] != K or b_all.shape[1:] != (N, RP) or b_all.shape[0] != a_all.shape[0]:
        raise ValueError("x [rows, K], y [rows, N], a_all [n_adapters, RP, K], b_all [n_adapters, N, RP]")
    nseg = seg_adapter.numel()
    rc = lib.kh_sgmv_fused_bf16(_ptr(x), _ptr(a_all), _ptr(b_all), _ptr(y), _ptr(seg_start), _ptr(seg_adapter),
                                _ptr(adapter_rank), _ptr(adapter_scale), nseg, max_seg_rows, N, K, RP, _stream())
    _lib.check(rc, "kh_sgmv_fused_bf16")
    return y


def sgmv_fused_grouped_table(ys, a_alls, b_alls) -> torch.Tensor:
    """The device table of sgmv_fused_grouped_: one row {a_all_l, b_all_l, y_l} of pointers per layer.  Build it once per
    set of layers; it holds addresses, so the tensors must stay where they are (and alive) while it is used."""
    if not (len(ys) == len(a_alls) == len(b_alls)) or not ys:
        raise ValueError("one y, a_all and b_all per layer")
    rows = []
    for y, a, b in zip(ys, a_alls, b_alls):
        _req(y, BF16, "y"); _req(a, BF16, "a_all"); _req(b, BF16, "b_all")
        if y.shape != ys[0].shape or a.shape != a_alls[0].shape or b.shape != b_alls[0].shape:
            raise ValueError("all layers of a grouped launch have the same shapes")
        rows.append([a.data_ptr(), b.data_ptr(), y.data_ptr()])
    return torch.tensor(rows, dtype=torch.int64, device=ys[0].device)


def sgmv_fused_grouped_(ys, x, a_alls, b_alls, seg_start, seg_adapter, adapter_rank, adapter_scale, max_seg_rows: int,
                        table: Optional[torch.Tensor] = None):
    """sgmv_fused_ for several layers that read the same x with the same segments (the to_k / to_v projections of all
    cross-attentions of one width) in ONE launch: ys[l][rows] += scale_a * bf16(x[rows] A_{l,a}^T) B_{l,a}^T.
    table: the result of sgmv_fused_grouped_table(ys, a_alls, b_alls) when the caller keeps it between calls."""
    lib = _lib.load()
    _req(x, BF16, "x"); _req(adapter_scale, torch.float32, "adapter_scale")
    for n, t in (("seg_start", seg_start), ("seg_adapter", seg_adapter), ("adapter_rank", adapter_rank)):
        _req(t, torch.int32, n)
    if table is None:
        table = sgmv_fused_grouped_table(ys, a_alls, b_alls)
    rows, K = x.shape
    N = ys[0].shape[1]
    RP = a_alls[0].shape[1]
    if (ys[0].shape[0] != rows or a_alls[0].shape[2] != K or b_alls[0].shape[1:] != (N, RP) or b_alls[0].shape[0] != a_alls[0].shape[0]
            or table.shape != (len(ys), 3) or table.dtype != torch.int64 or not table.is_cuda or not table.is_contiguous()):
        raise ValueError("x [rows, K], ys[l] [rows, N], a_alls[l] [n_adapters, RP, K], b_alls[l] [n_adapters, N, RP], table [layers, 3]")
    nseg = seg_adapter.numel()
    rc = lib.kh_sgmv_fused_grouped_bf16(_ptr(x), _ptr(table), len(ys), _ptr(seg_start), _ptr(seg_adapter), _ptr(adapter_rank),
                                        _ptr(adapter_scale), nseg, max_seg_rows, N, K, RP, _stream())
    _lib.check(rc, "kh_sgmv_fused_grouped_bf16")
    return ys


# --------------------------------------------------------------------------------------- K3
def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, heads: int, scale: Optional[float] = None,
              out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """softmax(q k^T * scale) v. q [B,T,H*64], k/v [B,S,H*64] (last-dim-contiguous views allowed)."""
    lib = _lib.load()
    B, T, inner = q.shape
    S = k.shape[1]
    hd = inner // heads
    for n, t in (("q", q), ("k", k), ("v", v)):
        if not t.is_cuda:
            raise _lib.KatzHipError(f"{n} must live on the GPU; katz_hip has no CPU path")
        if t.dtype != BF16 or t.stride(-1) != 1:
            raise TypeError(f"{n} must be bfloat16 with a contiguous last axis")
    if k.shape != (B, S, inner) or v.shape != (B, S, inner):
        raise ValueError("k and v must be [B,S,H*head_dim]")
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    if out is None:
        out = torch.empty((B, T, inner), dtype=BF16, device=q.device)
    if CALL_LOG is not None:
        CALL_LOG.append(("attention", B, heads, T, S, hd))
    rc = lib.kh_attention_bf16(_ptr(q), _ptr(k), _ptr(v), _ptr(out), B, heads, T, S, hd,
                               q.stride(1), k.stride(1), v.stride(1), out.stride(1),
                               q.stride(0), k.stride(0), v.stride(0), out.stride(0), float(scale), _stream())
    _lib.check(rc, "kh_attention_bf16")
    return out


# --------------------------------------------------------------------------------------- K4
_gn_workspace: dict = {}
_gn_retired: list = []     # outgrown workspaces, kept alive for graphs captured while they were current


_ws_slot: list = [0]


@contextlib.contextmanager
def side_branch():
    """Ops called inside this context take their shared scratch (the GroupNorm partial sums) from a second buffer, so
    that they may run on another stream beside ops called outside it."""
    _ws_slot[0] += 1
    try:
        yield
    finally:
        _ws_slot[0] -= 1


def _workspace(nbytes: int, device) -> torch.Tensor:
    """One grow-only fp32 scratch buffer per device and branch (allocated outside graph capture on first use)."""
    key = (device.type, device.index, _ws_slot[0])
    buf = _gn_workspace.get(key)
    if buf is None or buf.numel() * 4 < nbytes:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("katz_amd: run the step once eagerly before capturing it (the GroupNorm workspace grows "
                               "on first use and must outlive the graph)")
        if buf is not None:
            _gn_retired.append(buf)   # a captured graph may still write its partial sums there: never hand it back
        buf = torch.empty(max(nbytes // 4, 1 << 16), dtype=torch.float32, device=device)
        _gn_workspace[key] = buf
    return buf


def group_norm(x: torch.Tensor, num_groups: int, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor],
               eps: float, activation: str = "none", out: Optional[torch.Tensor] = None,
               add_nc: Optional[torch.Tensor] = None) -> torch.Tensor:
    """GroupNorm(+SiLU) of a 4-D [N,C,H,W] tensor, either contiguous (NCHW) or channels_last (NHWC
    memory); the output has the memory format of the input.  add_nc [N,C] (optional) is added to x
    per (sample, channel) before the statistics: norm(x + add_nc[:, :, None, None])."""
    lib = _lib.load()
    if activation not in ("none", "silu"):
        raise ValueError(f"unknown activation {activation!r}")  # the reference only printf's here
    if not x.is_cuda:
        raise _lib.KatzHipError("x must live on the GPU; katz_hip has no CPU path")
    if x.dtype != BF16 or x.dim() != 4:
        raise TypeError("group_norm expects a 4-D bfloat16 tensor")
    N, C, H, W = x.shape
    is_cl, is_cf = x.is_contiguous(memory_format=torch.channels_last), x.is_contiguous()
    if not (is_cl or is_cf):
        raise ValueError("x must be contiguous in NCHW or channels_last memory format")
    # both hold only when the two layouts coincide (C == 1 or H*W == 1): take whichever the kernels accept
    cl = 1 if (is_cl and (not is_cf or C % 8 == 0)) else 0
    if out is None:
        out = torch.empty_like(x)  # preserves the memory format
    elif out.stride() != x.stride() or out.dtype != BF16:
        raise ValueError("out must match x in dtype and strides")
    nbytes = lib.kh_group_norm_workspace_bytes(N, C, H * W, num_groups, cl)
    if nbytes < 0:
        _lib.check(int(nbytes), "kh_group_norm_workspace_bytes")
    ws = _workspace(int(nbytes), x.device)
    if add_nc is not None:
        _req(add_nc, BF16, "add_nc")
        if add_nc.shape != (N, C):
            raise ValueError(f"add_nc must be [N,C] = [{N},{C}], got {tuple(add_nc.shape)}")
    if CALL_LOG is not None:
        CALL_LOG.append(("group_norm", N, C, H * W))
    rc = lib.kh_group_norm_bf16(_ptr(x), _ptr(out), _ptr(weight), _ptr(bias), _ptr(add_nc), _ptr(ws), N, C, H * W, num_groups,
                                float(eps), 1 if activation == "silu" else 0, cl, _stream())
    _lib.check(rc, "kh_group_norm_bf16")
    return out


def layer_norm(x: torch.Tensor, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor], eps: float = 1e-5,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    lib = _lib.load()
    _req(x, BF16, "x")
    D = x.shape[-1]
    M = x.numel() // D
    if out is None:
        out = torch.empty_like(x)
    if CALL_LOG is not None:
        CALL_LOG.append(("layer_norm", M, D))
    rc = lib.kh_layer_norm_bf16(_ptr(x), _ptr(out), _ptr(weight), _ptr(bias), M, D, float(eps), _stream())
    _lib.check(rc, "kh_layer_norm_bf16")
    return out


# --------------------------------------------------------------------------------------- K5
def geglu(proj: torch.Tensor, approximate: str = "none") -> torch.Tensor:
    """value * gelu(gate) with [value | gate] = proj.chunk(2, -1)."""
    lib = _lib.load()
    _req(proj, BF16, "proj")
    D = proj.shape[-1] // 2
    M = proj.numel() // (2 * D)
    out = torch.empty(tuple(proj.shape[:-1]) + (D,), dtype=BF16, device=proj.device)
    rc = lib.kh_geglu_bf16(_ptr(proj), _ptr(out), M, D, 1 if approximate == "tanh" else 0, _stream())
    _lib.check(rc, "kh_geglu_bf16")
    return out


def gelu_mul(x: torch.Tensor, m: torch.Tensor, approximate: str = "tanh") -> torch.Tensor:
    """gelu(x) * m -- the argument order and tanh default of fast_kernel.fast_gelu_mul_fp16(x, m)."""
    lib = _lib.load()
    _req(x, BF16, "x"); _req(m, BF16, "m")
    if x.shape != m.shape:
        raise ValueError("x and m must have the same shape")
    out = torch.empty_like(x)
    rc = lib.kh_gelu_mul_bf16(_ptr(x), _ptr(m), _ptr(out), x.numel(), 1 if approximate == "tanh" else 0, _stream())
    _lib.check(rc, "kh_gelu_mul_bf16")
    return out


# --------------------------------------------------------------------------------------- residuals
def _ptr_array(ts: Sequence[torch.Tensor]):
    arr = (ctypes.c_void_p * max(len(ts), 1))()
    for i, t in enumerate(ts):
        arr[i] = t.data_ptr()
    return arr


def residual_add_(dst: torch.Tensor, residuals: Sequence[torch.Tensor]) -> torch.Tensor:
    """dst += mean_k(residuals[k]) in place (one residual: a plain add).  All tensors must share dst's
    memory layout."""
    lib = _lib.load()
    if not dst.is_cuda or dst.dtype != BF16:
        raise _lib.KatzHipError("dst must be a bfloat16 GPU tensor; katz_hip has no CPU path")
    for r in residuals:
        if r.shape != dst.shape or r.stride() != dst.stride() or r.dtype != BF16:
            raise ValueError("every residual must match dst in shape, strides and dtype")
    if CALL_LOG is not None:
        CALL_LOG.append(("residual_add", dst.numel(), len(residuals)))
    rc = lib.kh_residual_add_bf16(_ptr(dst), _ptr_array(residuals), len(residuals), 1.0 / len(residuals),
                                  dst.numel(), _stream())
    _lib.check(rc, "kh_residual_add_bf16")
    torch.autograd.graph.increment_version(dst)   # as an in-place torch op would: anything derived from dst is now stale
    return dst


def concat_residual(h: torch.Tensor, skip: torch.Tensor, residuals: Sequence[torch.Tensor] = ()) -> torch.Tensor:
    """cat([h, skip + mean_k residuals[k]], dim=1) for channels_last 4-D tensors."""
    lib = _lib.load()
    for n, t in (("h", h), ("skip", skip), *[("residual", r) for r in residuals]):
        if not t.is_cuda or t.dtype != BF16 or t.dim() != 4 or not t.is_contiguous(memory_format=torch.channels_last):
            raise ValueError(f"{n} must be a channels_last bfloat16 GPU tensor")
    N, C1, H, W = h.shape
    C2 = skip.shape[1]
    for r in residuals:
        if r.shape != skip.shape:
            raise ValueError("residuals must have the shape of skip")
    out = torch.empty((N, C1 + C2, H, W), dtype=BF16, device=h.device, memory_format=torch.channels_last)
    inv = 1.0 / len(residuals) if residuals else 1.0
    if CALL_LOG is not None:
        CALL_LOG.append(("concat_residual", N * H * W, C1, C2, len(residuals)))
    rc = lib.kh_concat_residual_bf16(_ptr(h), _ptr(skip), _ptr_array(residuals), len(residuals), inv, _ptr(out),
                                     N * H * W, C1, C2, _stream())
    _lib.check(rc, "kh_concat_residual_bf16")
    return out


def upsample_nearest2x(x: torch.Tensor) -> torch.Tensor:
    """F.interpolate(x, scale_factor=2.0, mode="nearest") for a channels_last bfloat16 [N,C,H,W] tensor."""
    lib = _lib.load()
    if not x.is_cuda or x.dtype != BF16 or x.dim() != 4 or not x.is_contiguous(memory_format=torch.channels_last):
        raise ValueError("x must be a channels_last bfloat16 GPU tensor")
    N, C, H, W = x.shape
    out = torch.empty((N, C, 2 * H, 2 * W), dtype=BF16, device=x.device, memory_format=torch.channels_last)
    rc = lib.kh_upsample_nearest2x_nhwc_bf16(_ptr(x), _ptr(out), N, H, W, C, _stream())
    _lib.check(rc, "kh_upsample_nearest2x_nhwc_bf16")
    return out


def pack_conv3x3_weight(weight: torch.Tensor) -> torch.Tensor:
    """nn.Conv2d weight [Cout,Cin,3,3] -> the [Cout,3,3,Cin] layout kh_conv3x3_nhwc_bf16 reads (a copy)."""
    if weight.dim() != 4 or weight.shape[2:] != (3, 3):
        raise ValueError("expected a [Cout,Cin,3,3] weight")
    return weight.detach().permute(0, 2, 3, 1).contiguous()


def conv3x3(x: torch.Tensor, w_packed: torch.Tensor, bias: Optional[torch.Tensor] = None, stride: int = 1,
            residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    """3x3 convolution, padding 1, of a channels_last [N,Cin,H,W] tensor; returns channels_last [N,Cout,Ho,Wo]
    (+ residual of that shape).  w_packed: pack_conv3x3_weight(weight)."""
    lib = _lib.load()
    if not x.is_cuda or x.dtype != BF16 or x.dim() != 4 or not x.is_contiguous(memory_format=torch.channels_last):
        raise ValueError("x must be a channels_last bfloat16 GPU tensor")
    Nb, Cin, H, W = x.shape
    Cout = w_packed.shape[0]
    if w_packed.shape != (Cout, 3, 3, Cin) or not w_packed.is_contiguous() or w_packed.dtype != BF16:
        raise ValueError("w_packed must be a contiguous bfloat16 [Cout,3,3,Cin] tensor")
    if bias is not None and (bias.shape != (Cout,) or bias.dtype != BF16 or not bias.is_contiguous()):
        raise ValueError("bias must be a contiguous bfloat16 [Cout] tensor")
    Ho, Wo = (H - 1) // stride + 1, (W - 1) // stride + 1
    out = torch.empty((Nb, Cout, Ho, Wo), dtype=BF16, device=x.device, memory_format=torch.channels_last)
    if residual is not None and (residual.shape != out.shape or residual.dtype != BF16
                                 or not residual.is_contiguous(memory_format=torch.channels_last)):
        raise ValueError("residual must be a channels_last bfloat16 tensor of the output's shape")
    if CALL_LOG is not None:
        CALL_LOG.append(("conv3x3", Nb * Ho * Wo, Cout, 9 * Cin, stride))
    _weight_prefetch_hint(w_packed)
    rc = lib.kh_conv3x3_nhwc_bf16(_ptr(x), _ptr(w_packed), _ptr(bias), _ptr(residual), _ptr(out), Nb, H, W, Cin, Cout,
                                  stride, _stream())
    _lib.check(rc, "kh_conv3x3_nhwc_bf16")
    return out


def conv3x3_gn_splits(x: torch.Tensor, cout: int, num_groups: int, stride: int = 1) -> int:
    """Row tiles per image of the GroupNorm statistics conv3x3_group_norm's convolution leaves for this input and output
    width, 0 when the shape is not taken (then: conv3x3 followed by group_norm)."""
    if not x.is_cuda or x.dtype != BF16 or x.dim() != 4:
        return 0
    Nb, Cin, H, W = x.shape
    return int(_lib.load().kh_conv3x3_gn_splits(Nb, H, W, Cin, cout, stride, num_groups))


def conv3x3_stats(x: torch.Tensor, w_packed: torch.Tensor, bias: Optional[torch.Tensor], num_groups: int,
                  add_nc: Optional[torch.Tensor] = None, residual: Optional[torch.Tensor] = None, stride: int = 1):
    """conv3x3(x, w_packed, bias, stride, residual) that also leaves the statistics of a GroupNorm(num_groups) of its result
    (+ add_nc per image and channel) as a by-product of its epilogue (kh_conv3x3_gn_stats_nhwc_bf16).  Returns
    (y, partials, splits): partials is a float [N, num_groups, splits, 2] tensor for group_norm_from_stats.  Only for
    shapes with conv3x3_gn_splits(...) > 0."""
    lib = _lib.load()
    if not x.is_cuda or x.dtype != BF16 or x.dim() != 4 or not x.is_contiguous(memory_format=torch.channels_last):
        raise ValueError("x must be a channels_last bfloat16 GPU tensor")
    Nb, Cin, H, W = x.shape
    Cout = w_packed.shape[0]
    if w_packed.shape != (Cout, 3, 3, Cin) or not w_packed.is_contiguous() or w_packed.dtype != BF16:
        raise ValueError("w_packed must be a contiguous bfloat16 [Cout,3,3,Cin] tensor")
    if bias is not None and (bias.shape != (Cout,) or bias.dtype != BF16 or not bias.is_contiguous()):
        raise ValueError("bias must be a contiguous bfloat16 [Cout] tensor")
    if add_nc is not None:
        add_nc = add_nc.reshape(Nb, Cout)
        if add_nc.dtype != BF16 or not add_nc.is_contiguous():
            raise ValueError("add_nc must be a contiguous bfloat16 [N,Cout] tensor")
    splits = int(lib.kh_conv3x3_gn_splits(Nb, H, W, Cin, Cout, stride, num_groups))
    if splits == 0:
        raise _lib.KatzHipError("kh_conv3x3_gn_stats_nhwc_bf16 does not take this shape (see conv3x3_gn_splits)")
    Ho, Wo = (H - 1) // stride + 1, (W - 1) // stride + 1
    out = torch.empty((Nb, Cout, Ho, Wo), dtype=BF16, device=x.device, memory_format=torch.channels_last)
    if residual is not None and (residual.shape != out.shape or residual.dtype != BF16
                                 or not residual.is_contiguous(memory_format=torch.channels_last)):
        raise ValueError("residual must be a channels_last bfloat16 tensor of the output's shape")
    partials = torch.empty((Nb, num_groups, splits, 2), dtype=torch.float32, device=x.device)
    if CALL_LOG is not None:
        CALL_LOG.append(("conv3x3", Nb * Ho * Wo, Cout, 9 * Cin, stride))
    _weight_prefetch_hint(w_packed)
    rc = lib.kh_conv3x3_gn_stats_nhwc_bf16(_ptr(x), _ptr(w_packed), _ptr(bias), _ptr(residual), _ptr(add_nc), _ptr(out),
                                           _ptr(partials), Nb, H, W, Cin, Cout, stride, num_groups, _stream())
    _lib.check(rc, "kh_conv3x3_gn_stats_nhwc_bf16")
    return out, partials, splits


def group_norm_from_stats(x: torch.Tensor, num_groups: int, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor],
                          eps: float, activation: str, partials: torch.Tensor, splits: int,
                          add_nc: Optional[torch.Tensor] = None) -> torch.Tensor:
    """group_norm(x, ..., add_nc=add_nc) as ONE launch, on the statistics conv3x3_stats left for x (+ the same add_nc):
    the norm's second pass alone (kh_group_norm_apply_bf16).  x: channels_last bfloat16 [N,C,H,W]."""
    lib = _lib.load()
    if not x.is_cuda or x.dtype != BF16 or x.dim() != 4 or not x.is_contiguous(memory_format=torch.channels_last):
        raise ValueError("x must be a channels_last bfloat16 GPU tensor")
    if activation not in ("none", "silu"):
        raise ValueError(f"unknown activation {activation!r}")
    N, C, H, W = x.shape
    for t_, name in ((weight, "weight"), (bias, "bias")):
        if t_ is not None and (t_.shape != (C,) or t_.dtype != BF16 or not t_.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous bfloat16 [C] tensor")
    if partials.dtype != torch.float32 or not partials.is_contiguous() or partials.numel() != N * num_groups * splits * 2:
        raise ValueError("partials must be the float [N, num_groups, splits, 2] tensor conv3x3_stats returned")
    if add_nc is not None:
        add_nc = add_nc.reshape(N, C)
        if add_nc.dtype != BF16 or not add_nc.is_contiguous():
            raise ValueError("add_nc must be a contiguous bfloat16 [N,C] tensor")
    out = torch.empty_like(x)
    if CALL_LOG is not None:
        CALL_LOG.append(("group_norm_apply", N, C, H * W))
    rc = lib.kh_group_norm_apply_bf16(_ptr(x), _ptr(out), _ptr(weight), _ptr(bias), _ptr(add_nc), _ptr(partials), splits, N, C,
                                      H * W, num_groups, float(eps), 1 if activation == "silu" else 0, _stream())
    _lib.check(rc, "kh_group_norm_apply_bf16")
    return out


def conv3x3_group_norm(x: torch.Tensor, w_packed: torch.Tensor, bias: Optional[torch.Tensor], num_groups: int,
                       gamma: Optional[torch.Tensor], beta: Optional[torch.Tensor], eps: float = 1e-5,
                       activation: str = "none", add_nc: Optional[torch.Tensor] = None, stride: int = 1) -> torch.Tensor:
    """group_norm(conv3x3(x, w_packed, bias), num_groups, gamma, beta, eps, activation, add_nc=add_nc) in two launches
    instead of three: conv3x3_stats, then group_norm_from_stats."""
    y, partials, splits = conv3x3_stats(x, w_packed, bias, num_groups, add_nc=add_nc, stride=stride)
    return group_norm_from_stats(y, num_groups, gamma, beta, eps, activation, partials, splits, add_nc=add_nc)


def cfg_euler_step(noise_pred: torch.Tensor, latents: torch.Tensor, coef: torch.Tensor, guidance_scale: float,
                   latents_out: Optional[torch.Tensor] = None, model_input_next: Optional[torch.Tensor] = None):
    """Guidance + Euler step (+ the next step's scaled, duplicated model input) in one kernel.
    noise_pred [2B,...] bf16 (uncond rows first), latents [B,...] bf16 or fp32, coef: fp32 GPU tensor
    {sigma, sigma_next, sqrt(sigma_next^2+1)}.  All tensors dense in one memory format (contiguous, or channels_last as
    the UNet returns its output).  latents_out may be latents itself.  Returns latents_out (allocated unless given)."""
    lib = _lib.load()
    if not noise_pred.is_cuda or noise_pred.dtype != BF16:
        raise _lib.KatzHipError("noise_pred must be a bfloat16 GPU tensor; katz_hip has no CPU path")

    def layout(t):   # the op is elementwise per batch row: every tensor must be dense in ONE memory format
        if t.is_contiguous():
            return "rows"
        if t.dim() == 4 and t.is_contiguous(memory_format=torch.channels_last):
            return "nhwc"
        return None

    kind = layout(noise_pred)
    if kind is None or noise_pred.numel() != 2 * latents.numel():
        raise ValueError("noise_pred must be dense (contiguous or channels_last) with twice the elements of latents")
    if latents.dtype not in (BF16, torch.float32) or not latents.is_cuda or layout(latents) != kind:
        raise ValueError("latents must be a bfloat16 or float32 GPU tensor in the memory format of noise_pred")
    if coef.dtype != torch.float32 or not coef.is_cuda or coef.numel() < 3:
        raise ValueError("coef must be a float32 GPU tensor of at least 3 elements")
    if latents_out is None:
        latents_out = torch.empty_like(latents)
    if latents_out.dtype != latents.dtype or latents_out.shape != latents.shape or layout(latents_out) != kind:
        raise ValueError("latents_out must match latents")
    if model_input_next is not None and (model_input_next.dtype != BF16 or layout(model_input_next) != kind
                                         or model_input_next.numel() != noise_pred.numel()):
        raise ValueError("model_input_next must be a bfloat16 tensor of noise_pred's size and memory format")
    rc = lib.kh_cfg_euler_step_bf16(_ptr(noise_pred), _ptr(latents), _ptr(latents_out), _ptr(model_input_next),
                                    latents.numel(), float(guidance_scale), _ptr(coef),
                                    1 if latents.dtype == torch.float32 else 0, _stream())
    _lib.check(rc, "kh_cfg_euler_step_bf16")
    return latents_out


def conv_out_cfg_euler(x: torch.Tensor, w_packed: torch.Tensor, bias: Optional[torch.Tensor], latents: torch.Tensor,
                       coef: torch.Tensor, guidance_scale: float, latents_out: Optional[torch.Tensor] = None,
                       model_input_next: Optional[torch.Tensor] = None, noise_pred_out: Optional[torch.Tensor] = None):
    """The tail of a denoising step in one launch: conv_out (4 output channels) on x [2B,C,H,W] channels_last, then
    guidance + Euler + the next step's scaled, duplicated input exactly as cfg_euler_step.  w_packed: [4,3,3,C]
    (pack_conv3x3_weight of the conv's weight).  latents [B,4,H,W] channels_last, bf16 or fp32; latents_out may be
    latents.  Returns latents_out."""
    lib = _lib.load()
    cl = torch.channels_last
    if not x.is_cuda or x.dtype != BF16 or x.dim() != 4 or not x.is_contiguous(memory_format=cl):
        raise ValueError("x must be a channels_last bfloat16 GPU tensor")
    NB, C, H, W = x.shape
    if NB % 2:
        raise ValueError("x holds guidance pairs: an even number of rows, unconditional rows first")
    Bl = NB // 2
    _req(w_packed, BF16, "w_packed")
    if tuple(w_packed.shape) != (4, 3, 3, C):
        raise ValueError(f"w_packed must be [4,3,3,{C}], got {tuple(w_packed.shape)}")
    if bias is not None:
        _req(bias, BF16, "bias")
    if (latents.dtype not in (BF16, torch.float32) or not latents.is_cuda or tuple(latents.shape) != (Bl, 4, H, W)
            or not latents.is_contiguous(memory_format=cl)):
        raise ValueError(f"latents must be a channels_last bfloat16 / float32 GPU tensor of shape {(Bl, 4, H, W)}")
    if latents_out is None:
        latents_out = torch.empty_like(latents)
    if latents_out.dtype != latents.dtype or latents_out.shape != latents.shape or not latents_out.is_contiguous(memory_format=cl):
        raise ValueError("latents_out must match latents")
    for name, t in (("model_input_next", model_input_next), ("noise_pred_out", noise_pred_out)):
        if t is not None and (t.dtype != BF16 or tuple(t.shape) != (NB, 4, H, W) or not t.is_contiguous(memory_format=cl)):
            raise ValueError(f"{name} must be a channels_last bfloat16 tensor of shape {(NB, 4, H, W)}")
    if coef.dtype != torch.float32 or not coef.is_cuda or coef.numel() < 3:
        raise ValueError("coef must be a float32 GPU tensor of at least 3 elements")
    rc = lib.kh_conv_out_cfg_euler_bf16(_ptr(x), _ptr(w_packed), _ptr(bias), _ptr(latents), _ptr(latents_out),
                                        _ptr(model_input_next), _ptr(noise_pred_out), Bl, H, W, C, float(guidance_scale),
                                        _ptr(coef), 1 if latents.dtype == torch.float32 else 0, _stream())
    _lib.check(rc, "kh_conv_out_cfg_euler_bf16")
    return latents_out


# --------------------------------------------------------------------------------------- per-launch timing
KERNEL_TAGS = {1: "lora_gemm", 2: "lora_gemm_f32", 3: "attention", 4: "group_norm_stats", 5: "group_norm_apply",
               6: "layer_norm", 7: "geglu", 8: "residual_add", 9: "concat_residual", 10: "sgmv_shrink",
               11: "sgmv_expand", 12: "lora_shrink", 13: "conv3x3", 14: "cfg_euler", 15: "upsample", 16: "lora_merge", 17: "conv_out_step", 18: "sgmv_fused"}


def profile_begin() -> None:
    """From now on every katz_hip launch carries its own HIP start/stop events (not graph-capturable)."""
    _lib.check(_lib.load().kh_profile_begin(), "kh_profile_begin")


def profile_end(capacity: int = 1 << 16):
    """Stop per-launch timing; returns [(kernel name, milliseconds)] in launch order (synchronises)."""
    tags = (ctypes.c_int32 * capacity)()
    ms = (ctypes.c_float * capacity)()
    n = _lib.load().kh_profile_end(tags, ms, capacity)
    if n < 0:
        _lib.check(-n, "kh_profile_end")
    n = min(n, capacity)
    return [(KERNEL_TAGS.get(tags[i], str(tags[i])), float(ms[i])) for i in range(n)]
