"""``moba_attn_varlen`` on MI355X: same signature and semantics as the reference
operator (moba/moba_efficient.py:270-443), computed by the hand-written HIP kernels of
``libmoba_hip.so``.  PyTorch owns every buffer; this module only validates arguments,
sizes workspaces and sequences the launches on the current stream.

Stages (each also callable on its own, which is how the tests reach them):
  chunk_mean        key chunk representatives         (moba_efficient.py:326-340)
  gate_topk         fp32 gate + causal top-k          (moba_efficient.py:341-371)
  build_lists       varlen gather lists               (moba_efficient.py:373-423)
  forward kernels   self + history attention + merge  (moba_efficient.py:69-183)
  backward kernels  dq, dk, dv                        (moba_efficient.py:185-267)
"""

from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

from . import _lib
from .plan import FWD_TILE_ROWS, MobaPlan, TILE_ROWS, make_plan

HEAD_DIM = 128
# MOBA_FIXED_REFERENCE=0 keeps the forward kernel on its running-maximum softmax for every problem (the
# fixed-reference form, with its redo list, is otherwise used where the C ABI's `redo` argument says)
FIXED_REFERENCE = os.environ.get("MOBA_FIXED_REFERENCE", "1") != "0"
# Dense prefixes (see MobaPlan.dense_local): None = where they pay (problems large enough for the kernels whose
# workgroups stay resident), True / False (MOBA_DENSE_PREFIX=1 / 0) = always / never.
DENSE_PREFIX = {"0": False, "1": True}.get(os.environ.get("MOBA_DENSE_PREFIX", ""))
# The per-slot partial results of a call take S * H * (K + 1) rows of head_dim elements, and the kernels index those
# rows with 32 bits.  A call whose partials would exceed this many bytes (MOBA_SCRATCH_GB, default 48), or 2^31
# rows, goes through its query heads in groups (whole key/value head groups): heads are independent, the result
# is the same bit for bit, and the scratch of one group is reused by the next.
SCRATCH_LIMIT_BYTES = int(float(os.environ.get("MOBA_SCRATCH_GB", "48")) * 2 ** 30)
# MOBA_DIRECT_ROWS=0 (a diagnostic): every row goes through its slot and the merge, also the rows without history slots
DIRECT_ROWS = os.environ.get("MOBA_DIRECT_ROWS", "1") != "0"
# diagnostics: with KEEP_SCRATCH set, a forward call leaves views of its scratch in last_scratch ("redo": the
# list of tiles the fixed-reference softmax handed to the kernel that tracks the maximum, count first; or None)
KEEP_SCRATCH = False
last_scratch = {}


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


# the current stream's handle without building a torch.cuda.Stream object (a few microseconds per stage otherwise)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device) -> ctypes.c_void_p:
    if _raw_stream is None:
        return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    index = device.index
    return ctypes.c_void_p(_raw_stream(torch.cuda.current_device() if index is None else index))


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return _lib.DTYPE_BF16
    if t.dtype == torch.float16:
        return _lib.DTYPE_F16
    raise TypeError("moba_attn_varlen supports bfloat16 and float16 q, k, v")


def _aligned(t: torch.Tensor) -> torch.Tensor:
    t = t.contiguous()
    return t if t.data_ptr() % 16 == 0 else t.clone()


def _dims(t: torch.Tensor):
    """(tokens, heads, head_dim) as the kernels see a [tokens, heads, head_dim] tensor or a batched
    [batch, heads, tokens, head_dim] one (the transformers layout: batch * tokens packed tokens)."""
    if t.dim() == 4:
        b, h, l, d = t.shape
        return b * l, h, d
    return tuple(t.shape)


def _row_strides(t: torch.Tensor):
    """(token stride, head stride) in elements; the stride of a dimension of size 1 means nothing and is
    replaced by the packed one."""
    if t.dim() == 4:
        b, H, S, D = t.shape
        return (t.stride(2) if S > 1 else D), (t.stride(1) if H > 1 else S * D)
    S, H, D = t.shape
    return (t.stride(0) if S > 1 else H * D), (t.stride(1) if H > 1 else D)


def _batch_stride(t: torch.Tensor):
    """(rows per batch entry, batch stride in elements) of a batched tensor; (0, 0) otherwise."""
    if t.dim() != 4 or t.shape[0] == 1:
        return 0, 0
    return t.shape[2], t.stride(0)


def _addressable(t: torch.Tensor) -> bool:
    """The kernels read 16 bytes per lane from rows of head_dim contiguous elements: any token and head
    strides that keep those reads aligned are read in place (a slice of a packed qkv projection, a
    [heads, tokens, head_dim] cache seen as [tokens, heads, head_dim], ...), as flash-attn does for
    the reference (moba/moba_efficient.py:89-128 hands such views straight to it)."""
    ts, hs = _row_strides(t)
    rows, bs = _batch_stride(t)
    return (t.stride(-1) == 1 and ts > 0 and hs > 0 and ts % 8 == 0 and hs % 8 == 0 and ts <= 1 << 23
            and (rows == 0 or (bs > 0 and bs % 8 == 0)) and t.data_ptr() % 16 == 0)


def _in_place(q, k, v):
    """q, k, v as the kernels will read them: untouched where addressable (k and v must share their
    strides), packed copies otherwise."""
    if not _addressable(q):
        q = _aligned(q)
    if not (_addressable(k) and _addressable(v) and _row_strides(k) == _row_strides(v)):
        k, v = _aligned(k), _aligned(v)
    return q, k, v


def _strides(q: Optional[torch.Tensor], k: Optional[torch.Tensor]):
    """The strides argument of the C ABI: {q token, q head, k/v token, k/v head, rows per batch entry,
    q batch, k/v batch} in elements (the last three 0 unless q, k are batched 4-D tensors)."""
    qs = _row_strides(q) if q is not None else (HEAD_DIM, HEAD_DIM)
    ks = _row_strides(k) if k is not None else (HEAD_DIM, HEAD_DIM)
    qr, qb = _batch_stride(q) if q is not None else (0, 0)
    kr, kb = _batch_stride(k) if k is not None else (0, 0)
    rows = qr or kr
    # (a tensor given alone stands for both: the entry point reads only its own entries)
    return (ctypes.c_int64 * 7)(qs[0], qs[1], ks[0], ks[1], rows, qb or kb if rows else 0, kb or qb if rows else 0)


def _check_qkv(q, k, v, gqa=False):
    if not (q.is_cuda and k.is_cuda and v.is_cuda):
        raise RuntimeError("moba_attn_varlen needs tensors on an AMD GPU (there is no CPU path)")
    if q.dtype not in (torch.bfloat16, torch.float16) or k.dtype != q.dtype or v.dtype != q.dtype:
        raise TypeError("moba_attn_varlen supports bfloat16 and float16 q, k, v (all three of the same dtype)")
    if q.dim() != 3 or k.shape != v.shape or k.dim() != 3 or q.shape[0] != k.shape[0] or q.shape[2] != k.shape[2]:
        raise ValueError("q must be [seqlen, heads, head_dim] and k, v [seqlen, kv_heads, head_dim]")
    if gqa:
        if k.shape[1] == 0 or q.shape[1] % k.shape[1] != 0:
            raise ValueError("the number of query heads must be a multiple of the number of key/value heads")
    elif q.shape != k.shape:
        raise ValueError("q, k, v must all be [seqlen, heads, head_dim] with the same number of heads")
    if not 0 < q.shape[2] <= HEAD_DIM:
        raise ValueError(f"head_dim must be at most {HEAD_DIM} (narrower heads are padded with zeros)")


# ----------------------------------------------------------------------------- stages
def chunk_mean(k: torch.Tensor, plan: MobaPlan, clear: Optional[torch.Tensor] = None) -> torch.Tensor:
    """kbar [F, H, D] in k's dtype: mean of K over every filtered chunk (exact sum, rounded once).
    `clear`: an int32 tensor the call zeroes on the way (the counts array of gate_topk)."""
    lib = _lib.load()
    S, H, D = _dims(k)
    if not _addressable(k):
        k = _aligned(k)
    kbar = torch.empty((plan.F, H, D), dtype=k.dtype, device=k.device)
    nbytes = lib.moba_chunk_mean_workspace_bytes(H, D, plan.F, plan.chunk_size)
    ws = torch.empty(nbytes // 8, dtype=torch.float64, device=k.device)
    _lib.check(lib.moba_chunk_mean(_ptr(k), _ptr(plan.tables["fchunk_tok"]), _ptr(kbar), _ptr(ws), S, H, D, plan.F,
                                   plan.chunk_size, _strides(None, k), _dtype_code(k), _ptr(clear),
                                   0 if clear is None else clear.numel(), _stream(k.device)),
               "moba_chunk_mean")
    return kbar


def gate_topk(q: torch.Tensor, kbar: torch.Tensor, plan: MobaPlan, return_scores: bool = False,
              cnt: Optional[torch.Tensor] = None):
    """sel [S, H, K] int32: selected filtered-chunk ids per (token, head), -1 padded (with a plan that has dense
    prefixes their tokens get no picks: the lists this selection feeds do not hold them).
    kbar may have fewer heads than q (grouped-query attention).  `cnt` (list_buffers()[0], zeroed): receives
    the counts build_lists starts from."""
    lib = _lib.load()
    S, H, D = _dims(q)
    Hkv = kbar.shape[1]
    if not _addressable(q):
        q = _aligned(q)
    sel = torch.empty((S, H, plan.K), dtype=torch.int32, device=q.device)
    scores = None
    if return_scores:
        scores = torch.full((S, H, plan.F), float("-inf"), dtype=torch.float32, device=q.device)
    _lib.check(lib.moba_gate_topk(_ptr(q), _ptr(kbar), _ptr(plan.tables["cu_seqlens"]), _ptr(plan.tables["seq_fbase"]),
                                  _ptr(sel), _ptr(scores), _ptr(plan.tables["pair_off"]), _ptr(cnt), S, H, Hkv, D,
                                  plan.nseq, plan.F, plan.chunk_size, plan.K, plan.dense_local, _strides(q, None),
                                  _dtype_code(q), _stream(q.device)), "moba_gate_topk")
    return (sel, scores) if return_scores else sel


def topk_from_scores(scores: torch.Tensor, K: int) -> torch.Tensor:
    """Selection stage alone on caller-supplied fp32 scores [S, H, F] (-inf = not a candidate)."""
    lib = _lib.load()
    S, H, F = scores.shape
    scores = scores.contiguous()
    sel = torch.empty((S, H, K), dtype=torch.int32, device=scores.device)
    _lib.check(lib.moba_topk_from_scores(_ptr(scores), _ptr(sel), S, H, F, K, _stream(scores.device)),
               "moba_topk_from_scores")
    return sel


def list_buffers(plan: MobaPlan, H: int, device, tile_rows: int = FWD_TILE_ROWS):
    """(cnt [P*H+1], seg_off [F*H+1], tile_off [F*H+1], seg_dest [M], tile_seg [tile bound]) int32, uninitialised:
    the arrays of build_lists, in one allocation (each start a multiple of 4 ints)."""
    sizes = [plan.P * H + 1, plan.F * H + 1, plan.F * H + 1, max(plan.pairs_per_head * H, 1),
             plan.hist_tile_bound(H, tile_rows)]
    starts = [0]
    for n in sizes:
        starts.append(starts[-1] + (n + 3) // 4 * 4)
    buf = torch.empty(starts[-1], dtype=torch.int32, device=device)
    return tuple(buf[a:a + n] for a, n in zip(starts, sizes))


def build_lists(sel: torch.Tensor, plan: MobaPlan, tile_rows: int = FWD_TILE_ROWS, buffers=None, counted=False,
                second_tile_rows: int = 0):
    """(seg_off [F*H+1], tile_off [F*H+1], seg_dest [M], tile_seg [tile bound]) int32 -- see csrc/lists.hip.
    The tile tables cut the lists into tiles of `tile_rows` rows (the forward kernel's by default).
    `buffers`: list_buffers() of the same plan, heads and tile_rows; `counted`: their cnt already holds the
    counts, left there by gate_topk; `second_tile_rows`: also return (tile_off, tile_seg) for tiles of that height."""
    lib = _lib.load()
    S, H, K = sel.shape
    dev = sel.device
    bound = plan.hist_tile_bound(H, tile_rows)
    cnt, seg_off, tile_off, seg_dest, tile_seg = buffers if buffers is not None else list_buffers(plan, H, dev, tile_rows)
    t = plan.tables
    second, second_args = (), (0, None, None, 0)
    if second_tile_rows:
        bound_b = plan.hist_tile_bound(H, second_tile_rows)
        second = (torch.empty(plan.F * H + 1, dtype=torch.int32, device=dev),
                  torch.empty(bound_b, dtype=torch.int32, device=dev))
        second_args = (second_tile_rows, _ptr(second[0]), _ptr(second[1]), bound_b)
    _lib.check(lib.moba_build_lists(_ptr(sel), _ptr(t["chunk_tok"]), _ptr(t["chunk_fb"]), _ptr(t["chunk_local"]),
                                    _ptr(t["pair_off"]), _ptr(cnt), _ptr(seg_off), _ptr(tile_off), _ptr(seg_dest),
                                    _ptr(tile_seg), S, H, K, plan.N, plan.F, plan.P, plan.cmax, tile_rows, bound,
                                    1 if counted else 0, *second_args, plan.dense_local, _stream(dev)),
               "moba_build_lists")
    return (seg_off, tile_off, seg_dest, tile_seg) + second


def tile_tables(seg_off: torch.Tensor, plan: MobaPlan, H: int, tile_rows: int):
    """(tile_off [F*H+1], tile_seg [tile bound]) for tiles of `tile_rows` rows, from the list starts."""
    lib = _lib.load()
    dev = seg_off.device
    tile_off = torch.empty(plan.F * H + 1, dtype=torch.int32, device=dev)
    bound = plan.hist_tile_bound(H, tile_rows)
    tile_seg = torch.empty(bound, dtype=torch.int32, device=dev)
    _lib.check(lib.moba_tile_tables(_ptr(seg_off), _ptr(tile_off), _ptr(tile_seg), H, plan.F, tile_rows, bound,
                                    _stream(dev)), "moba_tile_tables")
    return tile_off, tile_seg


class StageTimer:
    """Optional per-stage device timing: events are recorded on the launch stream around
    each stage, so reading them never perturbs the launches themselves."""

    def __init__(self, only=None):
        """only: names of the stages to time (a pair of event records costs the host some tens of
        microseconds, which shows in small problems); None = all."""
        self.events = {}
        self.only = None if only is None else set(only)

    def span(self, name, device):
        timer = self
        if self.only is not None and name not in self.only:
            return _NoSpan()

        class _Span:
            def __enter__(self_inner):
                self_inner.a = torch.cuda.Event(enable_timing=True)
                self_inner.b = torch.cuda.Event(enable_timing=True)
                self_inner.a.record(torch.cuda.current_stream(device))
                return self_inner

            def __exit__(self_inner, *exc):
                self_inner.b.record(torch.cuda.current_stream(device))
                timer.events.setdefault(name, []).append((self_inner.a, self_inner.b))
                return False

        return _Span()

    def ms(self):
        """stage -> list of elapsed milliseconds (call after a synchronize)."""
        return {k: [a.elapsed_time(b) for a, b in v] for k, v in self.events.items()}


class _NoSpan:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NO_SPAN = _NoSpan()


class _Geometry:
    """What a forward call needs besides its tensors, worked out once per (plan, heads, head_dim, element size):
    buffer sizes, the carving of the two scratch allocations, the key split and the tables' addresses."""

    def __init__(self, plan: MobaPlan, lib, H: int, D: int, esize: int):
        S, K = plan.S, plan.K
        self.tptr = {name: _ptr(t) for name, t in plan.tables.items()}
        self.null = ctypes.c_void_p(0)
        self.bound = plan.hist_tile_bound(H, FWD_TILE_ROWS)
        if plan.fallback:
            self.split = 1
        else:
            self.split = int(lib.moba_fwd_key_split(S, H, K, plan.chunk_size, self.bound, plan.fwd_self_tiles))
        # lists: cnt, seg_off, tile_off, seg_dest, tile_seg (int32, each start a multiple of 4 ints)
        sizes = [plan.P * H + 1, plan.F * H + 1, plan.F * H + 1, max(plan.pairs_per_head * H, 1), self.bound]
        self.list_sizes = sizes
        starts = [0]
        for n in sizes:
            starts.append(starts[-1] + (n + 3) // 4 * 4)
        self.list_starts = starts
        # ... and, for a call that a backward will follow, the backward kernels' tile tables behind them
        self.bwd_bound = plan.hist_tile_bound(H, TILE_ROWS)
        self.bwd_starts = [starts[-1], starts[-1] + (plan.F * H + 1 + 3) // 4 * 4]
        self.list_ints_with_bwd = self.bwd_starts[1] + self.bwd_bound
        # attention scratch: per-slot partial outputs, their log-sum-exps, the kernel's 8 tile counters, then
        # the list of tiles its fixed-reference softmax hands to the kernel that tracks the running maximum
        # (count first; the call zeroes the counters and the count)
        rows = S * H * (K + 1) * self.split
        self.rows = rows
        self.part_o_bytes = rows * D * esize
        self.scratch_ints = 8 + 1 + self.bound + plan.fwd_self_tiles * H
        self.ws_bytes = self.part_o_bytes + rows * 4 + self.scratch_ints * 4
        self.mean_ws = {}  # kv heads -> fp64 elements of the chunk mean's workspace
        self.bwd = {}      # kv heads -> sizes of the backward's scratch


def _geometry(plan: MobaPlan, lib, H: int, D: int, esize: int) -> _Geometry:
    key = (H, D, esize)
    g = plan.memo.get(key)
    if g is None:
        g = plan.memo[key] = _Geometry(plan, lib, H, D, esize)
    return g


def _forward(q, k, v, plan: MobaPlan, timer: Optional[StageTimer] = None, scale: float = 0.0, bwd_tables=None):
    """q, k, v: [tokens, heads, 128], or batched [batch, heads, tokens, 128] (read in place, see _dims), already
    addressable (_in_place).  Returns (out, lse, sel, seg_off, tile_off, seg_dest, tile_seg).
    bwd_tables: a list that receives the backward kernels' (tile_off, tile_seg), made on the way.
    The stages are those of chunk_mean(), gate_topk(), build_lists() above, called on precomputed sizes and
    addresses: at small shapes a forward is bound by the host's time per call."""
    lib = _lib.load()
    S, H, D = _dims(q)
    Hkv = _dims(k)[1]
    dev = q.device
    K = plan.K
    g = _geometry(plan, lib, H, D, q.element_size())
    tp, null = g.tptr, g.null
    span = (lambda name: timer.span(name, dev)) if timer is not None else (lambda name: _NO_SPAN)
    stream, code, strides = _stream(dev), _dtype_code(q), _strides(q, k)
    qp, kp, vp = _ptr(q), _ptr(k), _ptr(v)
    if plan.fallback:
        sel = seg_off = tile_off = seg_dest = tile_seg = None
        selp = seg_offp = tile_offp = seg_destp = tile_segp = null
    else:
        mean_ws = g.mean_ws.get(Hkv)
        if mean_ws is None:
            mean_ws = g.mean_ws[Hkv] = lib.moba_chunk_mean_workspace_bytes(Hkv, D, plan.F, plan.chunk_size) // 8
        kbar = torch.empty((plan.F, Hkv, D), dtype=q.dtype, device=dev)
        ws = torch.empty(mean_ws, dtype=torch.float64, device=dev)
        sel = torch.empty((S, H, K), dtype=torch.int32, device=dev)
        lists = torch.empty(g.list_starts[-1] if bwd_tables is None else g.list_ints_with_bwd, dtype=torch.int32,
                            device=dev)
        base = lists.data_ptr()
        if bwd_tables is None:
            bwd_args = (0, null, null, 0)
        else:
            b0, b1 = g.bwd_starts
            bwd_tables += [lists[b0:b0 + plan.F * H + 1], lists[b1:b1 + g.bwd_bound]]
            bwd_args = (TILE_ROWS, ctypes.c_void_p(base + 4 * b0), ctypes.c_void_p(base + 4 * b1), g.bwd_bound)
        cntp, seg_offp, tile_offp, seg_destp, tile_segp = (ctypes.c_void_p(base + 4 * a) for a in g.list_starts[:5])
        seg_off, tile_off, seg_dest, tile_seg = (lists[a:a + n] for a, n in zip(g.list_starts[1:5], g.list_sizes[1:]))
        selp, kbarp = _ptr(sel), _ptr(kbar)
        # the lists' counts are a by-product of the gate: the chunk mean clears the array, the gate adds to it
        with span("chunk_mean"):
            _lib.check(lib.moba_chunk_mean(kp, tp["fchunk_tok"], kbarp, _ptr(ws), S, Hkv, D, plan.F, plan.chunk_size,
                                           strides, code, cntp, g.list_sizes[0], stream), "moba_chunk_mean")
        with span("gate_topk"):
            _lib.check(lib.moba_gate_topk(qp, kbarp, tp["cu_seqlens"], tp["seq_fbase"], selp, null, tp["pair_off"],
                                          cntp, S, H, Hkv, D, plan.nseq, plan.F, plan.chunk_size, K, plan.dense_local,
                                          strides, code, stream), "moba_gate_topk")
        with span("build_lists"):
            _lib.check(lib.moba_build_lists(selp, tp["chunk_tok"], tp["chunk_fb"], tp["chunk_local"], tp["pair_off"],
                                            cntp, seg_offp, tile_offp, seg_destp, tile_segp, S, H, K, plan.N, plan.F,
                                            plan.P, plan.cmax, FWD_TILE_ROWS, g.bound, 1, *bwd_args, plan.dense_local,
                                            stream), "moba_build_lists")
    out = torch.empty((S, H, D), dtype=q.dtype, device=dev)
    lse = torch.empty((S, H), dtype=torch.float32, device=dev)
    ws2 = torch.empty(g.ws_bytes, dtype=torch.uint8, device=dev)
    base = ws2.data_ptr()
    part_op = ctypes.c_void_p(base)
    part_lsep = ctypes.c_void_p(base + g.part_o_bytes)
    queuesp = ctypes.c_void_p(base + g.part_o_bytes + g.rows * 4)
    redop = ctypes.c_void_p(base + g.part_o_bytes + g.rows * 4 + 32) if FIXED_REFERENCE else null
    if KEEP_SCRATCH:
        at = g.part_o_bytes + g.rows * 4 + 32
        last_scratch["redo"] = ws2[at:at + 4 * (g.scratch_ints - 8)].view(torch.int32) if FIXED_REFERENCE else None
    with span("fwd_partials"):
        _lib.check(lib.moba_fwd_partials(qp, kp, vp, part_op, part_lsep, seg_offp, tile_offp, seg_destp,
                                         tp.get("fchunk_tok", null), tp["achunk_tok"], tp["fwd_self_tile_prefix"],
                                         tile_segp, tp["fwd_self_tile_chunk"], tp["achunk_direct"] if DIRECT_ROWS else null,
                                         _ptr(out), _ptr(lse), S, H, Hkv, D, K, plan.F, plan.NA,
                                         plan.chunk_size, g.bound, plan.fwd_self_tiles, g.split, strides, queuesp,
                                         redop, scale, code, 0, 0, stream), "moba_fwd_partials")
    if not DIRECT_ROWS:
        with span("fwd_merge"):
            _lib.check(lib.moba_fwd_merge(part_op, part_lsep, selp, _ptr(out), _ptr(lse), S, H, D, K, g.split,
                                          null, null, 0, S, code, stream), "moba_fwd_merge")
    elif plan.merge_tokens:   # (the rows of every sequence's first attention chunk are written by the kernel above)
        with span("fwd_merge"):
            _lib.check(lib.moba_fwd_merge(part_op, part_lsep, selp, _ptr(out), _ptr(lse), S, H, D, K, g.split,
                                          tp["mrg_start"], tp["mrg_prefix"], plan.nseq, plan.merge_tokens, code,
                                          stream), "moba_fwd_merge")
    return out, lse, sel, seg_off, tile_off, seg_dest, tile_seg


def _backward(dout, q, k, v, out, lse, sel, seg_off, seg_dest, plan: MobaPlan, scale: float = 0.0, tables=None):
    """tables: the backward kernels' (tile_off, tile_seg) if the forward made them (made here otherwise)."""
    lib = _lib.load()
    S, H, D = _dims(q)
    Hkv = _dims(k)[1]
    dev = q.device
    K = plan.K
    g = _geometry(plan, lib, H, D, q.element_size())
    tp, null = g.tptr, g.null
    stream = _stream(dev)
    # One allocation for the call's scratch, every part a multiple of 16 bytes: the per-slot partial dQ, delta and
    # the log2 lse, the 16 tile counters of the two kernels (zeroed by the call), the backward kernels' own tile
    # tables (they cut the gather lists into tiles of their own height) and, for small problems, the fp32 sums of
    # the parts the dK/dV kernel cuts its key tiles into (0 bytes otherwise)
    b = g.bwd.get(Hkv)
    if b is None:
        bound = plan.hist_tile_bound(H, TILE_ROWS)
        kv_bytes = int(lib.moba_bwd_dkv_scratch_bytes(S, Hkv, plan.kv_tiles))
        # small problems: the keys of every history tile of the dQ kernel in `split` parts with slots of their own
        split = 1 if plan.fallback else int(lib.moba_bwd_dq_key_split(S, H, K, plan.chunk_size, bound, plan.self_tiles))
        sizes = [split * S * H * (K + 1) * D * q.element_size(), 2 * S * H * 4, 64,
                 0 if plan.fallback else (plan.F * H + 1) * 4, 0 if plan.fallback else bound * 4, kv_bytes]
        starts = [0]
        for n in sizes:
            starts.append(starts[-1] + (n + 15) // 16 * 16)
        b = g.bwd[Hkv] = (bound, kv_bytes, starts, split)
    bound, kv_bytes, starts, split = b
    ws = torch.empty(starts[-1], dtype=torch.uint8, device=dev)
    base = ws.data_ptr()
    part_dqp, deltap, queuesp, tile_offp, tile_segp, kvp = (ctypes.c_void_p(base + a) for a in starts[:6])
    if plan.fallback:
        tile_offp = tile_segp = null
    elif tables:
        tile_offp, tile_segp = _ptr(tables[0]), _ptr(tables[1])
    else:
        _lib.check(lib.moba_tile_tables(_ptr(seg_off), tile_offp, tile_segp, H, plan.F, TILE_ROWS, bound, stream),
                   "moba_tile_tables")
    dq = torch.empty((S, H, D), dtype=q.dtype, device=dev)  # packed, whatever the strides of q, k, v
    dk = torch.empty((S, Hkv, D), dtype=k.dtype, device=dev)
    dv = torch.empty((S, Hkv, D), dtype=v.dtype, device=dev)
    _lib.check(lib.moba_bwd(_ptr(dout), _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _ptr(sel), _ptr(seg_off),
                            tile_offp, _ptr(seg_dest), tp.get("fchunk_tok", null), tp["achunk_tok"],
                            tp["self_tile_prefix"], tile_segp, tp["self_tile_chunk"], tp.get("chunk_fid", null),
                            tp["chunk_tok"], tp["kv_tile_prefix"], tp["kv_tile_chunk"], tp["chunk_self_end"],
                            *((tp["achunk_direct"], tp["mrg_start"], tp["mrg_prefix"], plan.nseq, plan.merge_tokens)
                              if DIRECT_ROWS else (null, null, null, 0, S)),
                            deltap, part_dqp, _ptr(dq), _ptr(dk), _ptr(dv), S, H, Hkv, D, K, plan.F, plan.NA,
                            plan.chunk_size, bound, plan.self_tiles, plan.kv_tiles, split, _strides(q, k), queuesp,
                            kvp if kv_bytes else null, kv_bytes, scale, _dtype_code(q), stream), "moba_bwd")
    return dq, dk, dv


class _MobaAttention(torch.autograd.Function):
    """Counterpart of ``MixedAttention`` (moba/moba_efficient.py:67-267)."""

    @staticmethod
    def forward(ctx, q, k, v, plan, timer=None, scale=0.0):
        tables = []  # the backward's tile tables, made by the forward's list stage
        out, lse, sel, seg_off, _, seg_dest, _ = _forward(q, k, v, plan, timer, scale, bwd_tables=tables)
        ctx.plan = plan
        ctx.scale = scale
        ctx.aux = (sel, seg_off, seg_dest, tables)
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.mark_non_differentiable(lse)
        ctx.set_materialize_grads(False)  # no zero-filled gradient for lse on the way back
        return out, lse

    @staticmethod
    def backward(ctx, dout, _dlse):
        q, k, v, out, lse = ctx.saved_tensors
        sel, seg_off, seg_dest, tables = ctx.aux
        if dout is None:
            return None, None, None, None, None, None
        dq, dk, dv = _backward(_aligned(dout.to(q.dtype)), q, k, v, out, lse, sel, seg_off, seg_dest, ctx.plan, ctx.scale,
                               tables)
        if q.dim() == 4:   # gradients in the layout of the batched inputs: views of the packed results
            b, _, l, d = q.shape
            dq, dk, dv = (g.view(b, l, -1, d).transpose(1, 2) for g in (dq, dk, dv))
        return dq, dk, dv, None, None, None


def _choose_plan(plan: MobaPlan, H: int) -> MobaPlan:
    """The plan the kernels run: the batch's own, or its form with dense prefixes (MobaPlan.dense_local) where that
    pays -- when the forward kernel would still keep its workgroups resident, i.e. for problems of many tiles; on
    a problem of a few hundred tiles the long causal tiles of a dense prefix would run alone at the end."""
    if plan.fallback or plan.dense_local:
        return plan
    key = ("dense", H, DENSE_PREFIX)
    choice = plan.memo.get(key)
    if choice is None:
        choice = plan
        if DENSE_PREFIX is not False:
            dense = plan.with_dense_prefix()
            if dense.pairs_per_head == 0:
                # every token lies in a dense prefix: plain causal attention, no gate and no lists at all
                dense = make_plan(plan.cu, plan.chunk_size, 1, device=plan.device)
            if DENSE_PREFIX or _lib.load().moba_fwd_is_queued(dense.hist_tile_bound(H, FWD_TILE_ROWS),
                                                               dense.fwd_self_tiles, H):
                choice = dense
        plan.memo[key] = choice
    return choice


def _head_groups(plan: MobaPlan, H: int, Hkv: int, D: int, esize: int):
    """[(first query head, one past the last)]: the groups of heads a call works through, one group unless the
    per-slot partials of all heads together are too many (SCRATCH_LIMIT_BYTES, 2^31 slot rows)."""
    rep = H // Hkv
    rows_per_head = plan.S * (plan.K + 1)
    most = min((0x7fffffff - 1) // rows_per_head, SCRATCH_LIMIT_BYTES // (rows_per_head * (D * esize + 4)))
    most = max(rep, most // rep * rep)           # whole key/value head groups, at least one
    if most >= H:
        return [(0, H)]
    n = -(-H // most)                            # groups, as equal as whole key/value head groups allow
    size = -(-(H // rep) // n) * rep
    return [(h0, min(H, h0 + size)) for h0 in range(0, H, size)]


def _forward_in_groups(q, k, v, plan, groups, timer, scale, keep):
    """The forward group by group; `keep` receives what a backward needs of every group."""
    S, H, D = _dims(q)
    rep = H // _dims(k)[1]
    out = torch.empty((S, H, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((S, H), dtype=torch.float32, device=q.device)
    for h0, h1 in groups:
        group_plan = _choose_plan(plan, h1 - h0)
        tables = [] if keep is not None else None
        res = _forward(q[:, h0:h1], k[:, h0 // rep:h1 // rep], v[:, h0 // rep:h1 // rep], group_plan, timer, scale,
                       bwd_tables=tables)
        out[:, h0:h1] = res[0]
        lse[:, h0:h1] = res[1]
        if keep is not None:
            keep.append((group_plan, res[2], res[3], res[5], tables))
        del res
    return out, lse


class _MobaAttentionInGroups(torch.autograd.Function):
    """_MobaAttention for a call that works through its heads in groups (see SCRATCH_LIMIT_BYTES)."""

    @staticmethod
    def forward(ctx, q, k, v, plan, groups, timer=None, scale=0.0):
        keep = []
        out, lse = _forward_in_groups(q, k, v, plan, groups, timer, scale, keep)
        ctx.groups, ctx.keep, ctx.scale = groups, keep, scale
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.mark_non_differentiable(lse)
        ctx.set_materialize_grads(False)
        return out, lse

    @staticmethod
    def backward(ctx, dout, _dlse):
        q, k, v, out, lse = ctx.saved_tensors
        if dout is None:
            return None, None, None, None, None, None, None
        S, H, D = _dims(q)
        Hkv = _dims(k)[1]
        rep = H // Hkv
        dout = dout.to(q.dtype)
        dq = torch.empty((S, H, D), dtype=q.dtype, device=q.device)
        dk = torch.empty((S, Hkv, D), dtype=k.dtype, device=q.device)
        dv = torch.empty((S, Hkv, D), dtype=v.dtype, device=q.device)
        for (h0, h1), (group_plan, sel, seg_off, seg_dest, tables) in zip(ctx.groups, ctx.keep):
            g0, g1 = h0 // rep, h1 // rep
            got = _backward(_aligned(dout[:, h0:h1]), q[:, h0:h1], k[:, g0:g1], v[:, g0:g1], out[:, h0:h1].contiguous(),
                            lse[:, h0:h1].contiguous(), sel, seg_off, seg_dest, group_plan, ctx.scale, tables)
            dq[:, h0:h1], dk[:, g0:g1], dv[:, g0:g1] = got
            del got
        if q.dim() == 4:
            b, _, l, d = q.shape
            dq, dk, dv = (g.view(b, l, -1, d).transpose(1, 2) for g in (dq, dk, dv))
        return dq, dk, dv, None, None, None, None


def _attend(q, k, v, plan, timer=None, scale=0.0):
    """(out, lse): through autograd when a gradient may be asked for, straight to the kernels otherwise."""
    S, H, D = _dims(q)
    groups = _head_groups(plan, H, _dims(k)[1], D, q.element_size())
    grad = torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad)
    if len(groups) > 1:
        if grad:
            return _MobaAttentionInGroups.apply(q, k, v, plan, groups, timer, scale)
        return _forward_in_groups(q, k, v, plan, groups, timer, scale, None)
    plan = _choose_plan(plan, H)
    if grad:
        return _MobaAttention.apply(q, k, v, plan, timer, scale)
    return _forward(q, k, v, plan, timer, scale)[:2]


def moba_attn_varlen(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    cu_seqlens: torch.Tensor,
    max_seqlen: int,
    moba_chunk_size: int,
    moba_topk: int,
) -> torch.Tensor:
    """Mixture-of-block attention over a packed batch.

    Args (as moba/moba_efficient.py:270-297):
        q, k, v: [seqlen, heads, head_dim] bf16 or fp16, same number of heads
        cu_seqlens: int32 cumulative sequence lengths, starting at 0 and ending at seqlen
        max_seqlen: longest sequence (accepted for signature compatibility; sizes come from cu_seqlens)
        moba_chunk_size, moba_topk: block size and number of attended blocks (the current one included)
    Returns:
        [seqlen, heads, head_dim] in q's dtype.  Softmax scale is head_dim ** -0.5.

    The kernels are built for head_dim 128.  Narrower heads are padded with zeros to 128 (the scores, the
    gate and the softmax scale head_dim ** -0.5 are those of the narrow heads; the padding costs the work
    and memory of 128); wider heads are refused.
    """
    return moba_attn_varlen_with_lse(q, k, v, cu_seqlens, max_seqlen, moba_chunk_size, moba_topk)[0]


def moba_attn_varlen_gqa(q, k, v, cu_seqlens, max_seqlen, moba_chunk_size, moba_topk):
    """``moba_attn_varlen`` with grouped-query attention inside the operator: k, v are
    [seqlen, kv_heads, head_dim] and query head h reads key/value head h // (heads // kv_heads),
    as ``repeat_interleave`` on the head axis would give (moba/wrapper.py:59-61), without the
    copies.  The chunk representatives are computed once per key/value head; dk, dv are summed
    over the query heads of a group.  No counterpart in the reference operator."""
    return moba_attn_varlen_with_lse(q, k, v, cu_seqlens, max_seqlen, moba_chunk_size, moba_topk, gqa=True)[0]


def moba_attn_batched(query, key, value, moba_chunk_size, moba_topk):
    """The operator on the transformers layout: query [batch, heads, seqlen, head_dim], key and value
    [batch, kv_heads, seqlen, head_dim], every batch entry one sequence.  The tensors are read where they lie
    (no transposing copies, which ``hf_to_fa`` costs for batch > 1, moba/wrapper.py:56-58; no key/value head
    expansion); returns [batch * seqlen, heads, head_dim] like the packed operator.  Layouts the kernels cannot
    address, and head_dim below 128, go through packed copies."""
    from .wrapper import _cu_seqlens_for, hf_to_fa
    b, h, l, d = query.shape
    if key.shape != value.shape or key.dim() != 4 or key.shape[0] != b or key.shape[2] != l or key.shape[3] != d:
        raise ValueError("query must be [batch, heads, seqlen, head_dim] and key, value [batch, kv_heads, seqlen, head_dim]")
    cu_seqlens = _cu_seqlens_for(b, l, query.device)
    make_plan(cu_seqlens, moba_chunk_size, moba_topk, host_lengths=range(0, (b + 1) * l, l))
    in_place = (d == HEAD_DIM and _addressable(query) and _addressable(key) and _addressable(value)
                and _row_strides(key) == _row_strides(value) and _batch_stride(key) == _batch_stride(value))
    if not in_place:
        return moba_attn_varlen_gqa(hf_to_fa(query), hf_to_fa(key), hf_to_fa(value), cu_seqlens, l, moba_chunk_size,
                                    moba_topk)
    _check_qkv(query.select(0, 0).transpose(0, 1), key.select(0, 0).transpose(0, 1), value.select(0, 0).transpose(0, 1),
               gqa=True)
    plan = make_plan(cu_seqlens, moba_chunk_size, moba_topk, device=query.device)
    return _attend(query, key, value, plan)[0]


# lets moba_layer skip the key/value head expansion when it drives this operator
moba_attn_varlen.grouped_query_impl = moba_attn_varlen_gqa
# ... and the transposing copies of a batch of more than one sequence
moba_attn_varlen.batched_impl = moba_attn_batched
# ... and tells it that make_plan(host_lengths=...) spares the device-to-host read of cu_seqlens
moba_attn_varlen.takes_host_lengths = True
moba_attn_varlen_gqa.takes_host_lengths = True


def moba_attn_varlen_with_lse(q, k, v, cu_seqlens, max_seqlen, moba_chunk_size, moba_topk, timer=None, gqa=False):
    """As ``moba_attn_varlen`` but also returns the natural-log LSE [seqlen, heads] fp32.
    ``timer`` (a StageTimer) collects per-stage device times; ``gqa`` allows fewer key/value heads."""
    _check_qkv(q, k, v, gqa)
    plan = make_plan(cu_seqlens, moba_chunk_size, moba_topk, device=q.device)
    if plan.S != q.shape[0]:
        raise ValueError(f"cu_seqlens ends at {plan.S} but q has {q.shape[0]} tokens")
    head_dim = q.shape[2]
    if head_dim < HEAD_DIM:
        pad = (0, HEAD_DIM - head_dim)
        q, k, v = (torch.nn.functional.pad(x, pad) for x in (q, k, v))
        out, lse = _attend(q, k, v, plan, timer, head_dim ** -0.5)
        return out[..., :head_dim].contiguous(), lse
    q, k, v = _in_place(q, k, v)
    return _attend(q, k, v, plan, timer)
