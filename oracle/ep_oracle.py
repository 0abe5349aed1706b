"""CPU oracle for the EPBuffer dispatch/combine hot path.

TEST INFRASTRUCTURE ONLY.  This module is the checker the HIP path is compared
against; only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
import it.  The product (the deep_ep package and libdeep_ep_hip.so) never does.

It restates, on the CPU with numpy (integer / byte work) and torch-CPU (BF16 and
FP8 e4m3fn arithmetic, which the reference itself delegates to torch), what the
reference computes on this path.  Every function cites the reference lines it
follows (paths relative to the reference root).

Pinning status of each function (what independent evidence fixes its results):

* send_layout / recv_layout / expand   -- integer exact.  Pinned by a sequential
  simulation of the device kernels written independently in tests/, by the worked
  two-rank example derived by hand from the kernels, and by the invariants the
  reference's own test asserts (tests/ep/test_ep.py:182-296).
* token_layout / buffer sizes           -- pinned by the byte counts that follow from
  deep_ep/include/deep_ep/layout/ep/token.hpp:24-45 (7488 / 14432 / 14464 / 14368).
* quantise                              -- pinned by golden vectors produced from the
  reference's own deep_ep/utils/math.py (tests/golden/), by closed forms
  (power-of-two amax, all-zero groups, +-amax -> 0x7E/0xFE) and by an independent
  integer re-implementation of the e4m3fn rounding.
* no_sync_sizes                         -- pinned by the literal row counts that follow from
  csrc/buffers/ep.hpp:288,316-320 at the headline shape (130 816 rows with one partition,
  3 146 752 with 32), a case worked by hand, and a brute-force check that it bounds every
  layout of random tiny routings.
* combine_weighted (an extension)       -- pinned by a per-element numpy-float32 loop over slots
  derived from the closed form, and by reducing to the plain combine when every weight is 1.
* combine_partial / combine_final       -- pinned by golden vectors produced from the
  reference's own deep_ep/utils/refs.py combine (tests/golden/), by exact cases
  (K=1 identity, powers of two) and by an independent numpy-float32 loop in tests/.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

UB_ALIGN = 32                 # deep_ep/include/deep_ep/common/compiled.hpp:39
ALLOC_ALIGN = 2097152         # deep_ep/include/deep_ep/common/compiled.hpp:48
SF_PACK_BYTES = 2             # sf_pack_t = int16_t, compiled.hpp:33
FP8_MAX = 448.0


def ceil_div(a: int, b: int) -> int:
    return (a + b - 1) // b


def align(a: int, b: int) -> int:
    # deep_ep/utils/math.py:26-27, deep_ep/include/deep_ep/common/math.hpp:29-32
    return ceil_div(a, b) * b


# --------------------------------------------------------------------------------------
# Token / buffer layout  (deep_ep/include/deep_ep/layout/ep/token.hpp:9-130)
# --------------------------------------------------------------------------------------
@dataclass(frozen=True)
class TokenLayout:
    num_hidden_bytes: int
    num_sf_bytes: int
    num_topk: int
    with_metadata: bool = True

    @property
    def num_metadata_bytes(self) -> int:
        # token.hpp:24-25
        n = self.num_topk * 4
        if self.with_metadata:
            n += align(self.num_topk * 8, UB_ALIGN) + 4
        return n

    def num_bytes(self, skip_hidden: bool = False) -> int:
        # token.hpp:36-43
        n = 0 if skip_hidden else self.num_hidden_bytes
        if self.num_sf_bytes > 0:
            n += align(self.num_sf_bytes, UB_ALIGN)
        return n + align(self.num_metadata_bytes, UB_ALIGN)

    @property
    def sf_offset(self) -> int:
        return align(self.num_hidden_bytes, UB_ALIGN)            # token.hpp:60-62

    @property
    def topk_idx_offset(self) -> int:
        if self.num_sf_bytes > 0:                                 # token.hpp:65-69
            return self.sf_offset + align(self.num_sf_bytes, UB_ALIGN)
        return self.num_hidden_bytes

    @property
    def topk_weights_offset(self) -> int:
        off = self.topk_idx_offset                                # token.hpp:72-77
        if self.with_metadata:
            off += align(8 * self.num_topk, UB_ALIGN)
        return off

    @property
    def src_token_global_idx_offset(self) -> int:
        return self.topk_weights_offset + 4 * self.num_topk      # token.hpp:80-82


def dispatch_token_layout(num_hidden_bytes: int, num_sf_packs: int, num_topk: int,
                          cached: bool = False) -> TokenLayout:
    # csrc/kernels/ep/dispatch.hpp:13-18; cached mode drops idx+src (dispatch_copy_epilogue.hpp:226)
    return TokenLayout(num_hidden_bytes, num_sf_packs * SF_PACK_BYTES, num_topk, not cached)


def combine_token_layout(hidden: int, num_topk: int) -> TokenLayout:
    # csrc/kernels/ep/combine.hpp:14-16
    return TokenLayout(hidden * 2, 0, num_topk, False)


def dispatch_buffer_size(max_tokens: int, hidden: int, num_sf_packs: int, num_topk: int,
                         elem_size: int, num_ranks: int) -> int:
    # csrc/buffers/ep.hpp:560-569
    return num_ranks * max_tokens * dispatch_token_layout(hidden * elem_size, num_sf_packs, num_topk).num_bytes()


def combine_buffer_size(num_ranks: int, max_tokens: int, hidden: int, num_topk: int) -> int:
    # csrc/buffers/ep.hpp:571-579
    return min(num_topk, num_ranks) * max_tokens * combine_token_layout(hidden, num_topk).num_bytes()


def calculate_buffer_size(num_ranks: int, max_tokens: int, hidden: int, num_topk: int, use_fp8: bool) -> int:
    # csrc/buffers/ep.hpp:581-605
    assert num_ranks > 0 and max_tokens > 0 and hidden > 0 and num_topk >= 0
    num_topk = 32 if num_topk == 0 else num_topk
    packs = ceil_div(hidden, 32) if use_fp8 else 0
    d = dispatch_buffer_size(max_tokens, hidden, packs, num_topk, 1 if use_fp8 else 2, num_ranks)
    c = combine_buffer_size(num_ranks, max_tokens, hidden, num_topk)
    return align(max(d, c), ALLOC_ALIGN)


# --------------------------------------------------------------------------------------
# Quantiser  (deep_ep/utils/math.py:30-38)
# --------------------------------------------------------------------------------------
def quantise(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """BF16 [T,H] -> (e4m3fn payload as uint8 [T,H], fp32 scales [T, ceil(H/128)]).

    Per (row, 128-channel group): amax over |x| in fp32 clamped below at 1e-4; payload
    = RNE_e4m3fn( f32(x) * inv ), scale = amax / 448 (fp32 IEEE division).  math.py:33-38.
    `inv` is what torch makes of the reference's `448.0 / amax_tensor`: Tensor.__rtruediv__
    evaluates it as amax.reciprocal() * 448.0, i.e. fl(fl(1/amax) * 448) with two fp32
    roundings, which differs from a single division in the last bit for some amax (the golden
    vectors from the reference's math.py pin this).
    """
    assert x.dim() == 2 and x.dtype == torch.bfloat16
    m, n = x.shape
    an = align(n, 128)
    xp = torch.nn.functional.pad(x, (0, an - n), value=0).view(m, -1, 128)
    amax = xp.abs().float().amax(dim=2).view(m, -1).clamp(1e-4)
    q = (xp.float() * (FP8_MAX / amax.unsqueeze(2))).to(torch.float8_e4m3fn)
    q = q.view(m, an)[:, :n].contiguous()
    return q.view(torch.uint8), (amax / FP8_MAX).view(m, -1)


# --------------------------------------------------------------------------------------
# Send side: dedup per destination rank, slot assignment, counts
# (deep_ep/include/deep_ep/impls/ep/dispatch.hpp:153-293; dedup common/simt.hpp:24-34)
# --------------------------------------------------------------------------------------
def send_layout(topk_idx: np.ndarray, num_experts: int, num_ranks: int):
    """Returns (dst_buffer_slot_idx [T,K] i32, num_send_per_rank [R] i32, expert_hist [E] i32).

    A (t, j) entry is a *master* iff e >= 0 and no higher j of the same token maps to the
    same destination rank (dispatch.hpp:180-181).  Masters get consecutive slots in the
    destination's region in ascending token order -- the deterministic choice among the
    arrival orders the reference's atomics allow (dispatch.hpp:184-189,267-276).
    """
    topk_idx = np.asarray(topk_idx, dtype=np.int64)
    T, K = topk_idx.shape
    epr = num_experts // num_ranks
    valid = topk_idx >= 0
    rank = np.where(valid, topk_idx // epr, -1)
    master = valid.copy()
    for j in range(K):
        for jj in range(j + 1, K):
            master[:, j] &= ~(valid[:, jj] & (rank[:, jj] == rank[:, j]))
    dst = np.full((T, K), -1, dtype=np.int32)
    cnt = np.zeros(num_ranks, dtype=np.int32)
    for r in range(num_ranks):
        m = master & (rank == r)                 # at most one per token
        hit = m.any(axis=1)
        order = np.cumsum(hit) - 1
        tt, jj = np.nonzero(m)
        dst[tt, jj] = order[tt]
        cnt[r] = int(hit.sum())
    hist = np.bincount(topk_idx[valid].ravel(), minlength=num_experts).astype(np.int32)
    return dst, cnt, hist


def pack_regions(x_bytes: np.ndarray, sf_bytes: Optional[np.ndarray], topk_idx: np.ndarray,
                 topk_weights: Optional[np.ndarray], dst_slot: np.ndarray, num_send_per_rank: np.ndarray,
                 num_experts: int, num_ranks: int, src_rank: int, max_tokens: int,
                 cached: bool = False) -> List[np.ndarray]:
    """Packed rows per destination rank: list of [cnt_r, token_bytes] uint8.

    Row = hidden bytes || SF bytes (32-aligned) || metadata: all K topk_idx (i64, padded to
    32 B), all K topk_weights (f32), src_token_global_idx = src_rank*max_tokens + t
    (dispatch.hpp:768-794,777; token.hpp).  Cached mode carries only the weights.
    """
    T, K = topk_idx.shape
    HB = x_bytes.shape[1]
    SB = 0 if sf_bytes is None else sf_bytes.shape[1]
    lay = TokenLayout(HB, SB, K, not cached)
    epr = num_experts // num_ranks
    out = [np.zeros((int(num_send_per_rank[r]), lay.num_bytes()), dtype=np.uint8) for r in range(num_ranks)]
    w = (np.zeros((T, K), np.float32) if topk_weights is None else np.asarray(topk_weights, np.float32))
    for t in range(T):
        for j in range(K):
            s = int(dst_slot[t, j])
            if s < 0:
                continue
            r = int(topk_idx[t, j]) // epr
            row = out[r][s]
            row[:HB] = x_bytes[t]
            if SB:
                row[lay.sf_offset:lay.sf_offset + SB] = sf_bytes[t]
            if not cached:
                row[lay.topk_idx_offset:lay.topk_idx_offset + 8 * K] = topk_idx[t].astype('<i8').view(np.uint8)
                row[lay.src_token_global_idx_offset:lay.src_token_global_idx_offset + 4] = \
                    np.array([src_rank * max_tokens + t], '<i4').view(np.uint8)
            row[lay.topk_weights_offset:lay.topk_weights_offset + 4 * K] = w[t].astype('<f4').view(np.uint8)
    return out


# --------------------------------------------------------------------------------------
# Receive side: counts, aligned expert starts, expand slots, metadata
# (dispatch.hpp:449-546, dispatch_copy_epilogue.hpp:265-283,397-429,450-545; deterministic
#  order of deep_ep/buffers/ep.py:100-160)
# --------------------------------------------------------------------------------------
def recv_layout(recv_topk_idx: np.ndarray, recv_src_global: np.ndarray, num_recv_per_rank: Sequence[int],
                num_experts: int, num_ranks: int, rank_idx: int, expert_alignment: int):
    """`recv_topk_idx` [N,K] = the *global* expert ids of the receive stream (region of source
    rank 0 first, then 1, ...; within a region in slot order).  Returns a dict with the handle
    tensors.  Slots inside an expert follow the stream order then j, which -- because regions
    are filled in ascending token order -- is ascending src_token_global_idx, i.e. the layout
    EPHandle.deterministic_sort produces.
    """
    recv_topk_idx = np.asarray(recv_topk_idx, dtype=np.int64)
    N, K = recv_topk_idx.shape
    epr = num_experts // num_ranks
    A = expert_alignment
    local = recv_topk_idx - rank_idx * epr
    is_local = (recv_topk_idx >= 0) & (local >= 0) & (local < epr)
    cnt = np.bincount(local[is_local].ravel(), minlength=epr).astype(np.int32)      # dispatch.hpp:475-481
    aligned = (cnt + A - 1) // A * A
    start = np.concatenate([[0], np.cumsum(aligned)[:-1]]).astype(np.int64)          # copy_epilogue.hpp:265-277,426
    psum_expert = (start + cnt).astype(np.int32)                                      # dispatch.hpp:504-521
    psum_rank = np.cumsum(np.asarray(num_recv_per_rank, dtype=np.int64)).astype(np.int32)  # :524-545
    # stable rank of each (i, j) among entries with the same local expert, in (i, j) order
    flat_e = np.where(is_local, local, epr).ravel()
    order = np.argsort(flat_e, kind='stable')
    rank_in_e = np.empty(N * K, dtype=np.int64)
    sorted_e = flat_e[order]
    first = np.searchsorted(sorted_e, sorted_e, side='left')
    rank_in_e[order] = np.arange(N * K) - first
    slots = np.where(is_local.ravel(), start[np.minimum(flat_e, epr - 1)] + rank_in_e, -1).reshape(N, K)
    jj = np.arange(K)[None, :]
    master = np.where(is_local, jj, -1).max(axis=1) if N else np.zeros(0, np.int64)   # copy_epilogue.hpp:486,521
    meta = np.concatenate([slots, np.asarray(recv_src_global, np.int64).reshape(N, 1),
                           master.reshape(N, 1)], axis=1).astype(np.int32)            # :514-522
    return dict(
        num_unaligned_recv_tokens_per_expert=cnt,
        psum_num_recv_tokens_per_expert=psum_expert,
        psum_num_recv_tokens_per_rank=psum_rank,
        recv_src_metadata=meta,
        num_recv_tokens=int(N),
        num_expanded_tokens=int(aligned.sum()),                 # csrc/buffers/ep.hpp:308-315
        num_recv_tokens_per_expert_list=[int(v) for v in aligned],
        expert_start=start.astype(np.int32),
    )


def expand(recv_rows_hidden: np.ndarray, recv_rows_sf: Optional[np.ndarray], recv_rows_weights: Optional[np.ndarray],
           meta: np.ndarray, num_expanded: int):
    """Copy each received row to every slot listed in its metadata row; everything else
    (the alignment padding) is zero.  dispatch_copy_epilogue.hpp:471-512,547-620."""
    N, K2 = meta.shape
    K = K2 - 2
    rx = np.zeros((num_expanded, recv_rows_hidden.shape[1]), dtype=recv_rows_hidden.dtype)
    rs = None if recv_rows_sf is None else np.zeros((num_expanded, recv_rows_sf.shape[1]), dtype=recv_rows_sf.dtype)
    rw = None if recv_rows_weights is None else np.zeros((num_expanded,), dtype=np.float32)
    for j in range(K):
        s = meta[:, j]
        m = s >= 0
        rx[s[m]] = recv_rows_hidden[m]
        if rs is not None:
            rs[s[m]] = recv_rows_sf[m]
        if rw is not None:
            rw[s[m]] = recv_rows_weights[m, j]
    return rx, rs, rw


def no_sync_sizes(num_ranks: int, max_tokens: int, num_topk: int, num_experts: int, expert_alignment: int):
    # csrc/buffers/ep.hpp:288,316-320
    epr = num_experts // num_ranks
    n_exp = num_ranks * max_tokens * min(num_topk, epr) + (expert_alignment - 1) * epr
    return num_ranks * max_tokens, align(n_exp, expert_alignment)


# --------------------------------------------------------------------------------------
# One GPU's share: source rank == rank_idx is the only sender (what the HIP path computes)
# --------------------------------------------------------------------------------------
def rank_share_layout(topk_idx: np.ndarray, num_experts: int, num_ranks: int, rank_idx: int,
                      expert_alignment: int, max_tokens: int):
    topk_idx = np.asarray(topk_idx, dtype=np.int64)
    dst, cnt_send, hist = send_layout(topk_idx, num_experts, num_ranks)
    epr = num_experts // num_ranks
    lo, hi = rank_idx * epr, (rank_idx + 1) * epr
    hits = ((topk_idx >= lo) & (topk_idx < hi)).any(axis=1)
    toks = np.nonzero(hits)[0]
    per_rank = np.zeros(num_ranks, dtype=np.int64)
    per_rank[rank_idx] = len(toks)
    out = recv_layout(topk_idx[toks], rank_idx * max_tokens + toks, per_rank,
                      num_experts, num_ranks, rank_idx, expert_alignment)
    out.update(dst_buffer_slot_idx=dst, dst_gsge_idx=np.full_like(dst, -1),
               num_send_tokens_per_rank=cnt_send, expert_hist=hist, recv_token_idx=toks)
    return out


def rank_share_dispatch(x_rows: np.ndarray, sf_rows: Optional[np.ndarray], topk_weights: Optional[np.ndarray],
                        lay: dict):
    """Expanded outputs of one rank's own tokens given `rank_share_layout`'s result."""
    toks = lay['recv_token_idx']
    w = None if topk_weights is None else np.asarray(topk_weights, np.float32)[toks]
    return expand(x_rows[toks], None if sf_rows is None else sf_rows[toks], w,
                  lay['recv_src_metadata'], lay['num_expanded_tokens'])


# --------------------------------------------------------------------------------------
# Combine  (impls/ep/combine.hpp:80-106,291-324; combine_utils.hpp:14-93;
#           combine_reduce_epilogue.hpp:96-154; oracle deep_ep/utils/refs.py:157-247)
# --------------------------------------------------------------------------------------
def _ordered_sum_bf16(rows: List[torch.Tensor], hidden: int) -> torch.Tensor:
    """fp32 left-to-right sum of BF16 rows, rounded once to BF16 (combine_utils.hpp:56-92).
    0 rows -> zeros (:24-28); 1 row -> verbatim (:29-37)."""
    if len(rows) == 0:
        return torch.zeros(hidden, dtype=torch.bfloat16)
    if len(rows) == 1:
        return rows[0].clone()
    acc = rows[0].float()
    for r in rows[1:]:
        acc = acc + r.float()
    return acc.to(torch.bfloat16)


def combine_partial(y: torch.Tensor, expanded_weights: Optional[torch.Tensor], meta: np.ndarray,
                    num_ranks: int, rank_idx: int, max_tokens: int):
    """Owner-side reduce of every received token (combine.hpp:291-324).

    Returns (partials: dict[(group, src_global_idx)] -> BF16 [H], weight vectors: same keys -> f32 [K]).
    group = master_j when num_ranks >= K else the owner's rank id (combine.hpp:98-103,301-307).
    """
    N, K2 = meta.shape
    K = K2 - 2
    H = y.shape[1]
    parts, wvecs = {}, {}
    for i in range(N):
        slots = [int(s) for s in meta[i, :K] if s >= 0]
        p = _ordered_sum_bf16([y[s] for s in slots], H)
        group = rank_idx if num_ranks < K else int(meta[i, K + 1])
        key = (group, int(meta[i, K]))
        parts[key] = p
        if expanded_weights is not None:
            wv = torch.zeros(K, dtype=torch.float32)
            for j in range(K):
                if meta[i, j] >= 0:
                    wv[j] = expanded_weights[int(meta[i, j])]
            wvecs[key] = wv
    return parts, wvecs


def combine_final(topk_idx: np.ndarray, num_experts: int, num_ranks: int, src_rank: int, max_tokens: int,
                  partial_of, weights_of, bias_0: Optional[torch.Tensor], bias_1: Optional[torch.Tensor],
                  hidden: int, with_weights: bool):
    """Token-owner reduce (combine_reduce_epilogue.hpp:96-154): masters = last valid j per
    destination rank; inputs = bias_0, bias_1, partials in ascending master j, summed
    left-to-right in fp32 and rounded once (a single input is copied verbatim).  Weight
    vectors of the masters are OR-merged bitwise (:19-43,141-153)."""
    topk_idx = np.asarray(topk_idx, dtype=np.int64)
    T, K = topk_idx.shape
    epr = num_experts // num_ranks
    out = torch.zeros((T, hidden), dtype=torch.bfloat16)
    wout = np.zeros((T, K), dtype=np.uint32) if with_weights else None
    for t in range(T):
        seen = set()
        masters = []
        for j in range(K - 1, -1, -1):
            e = int(topk_idx[t, j])
            if e < 0:
                continue
            r = e // epr
            if r not in seen:
                masters.append(j)
            seen.add(r)
        masters.sort()
        rows = []
        if bias_0 is not None:
            rows.append(bias_0[t])
        if bias_1 is not None:
            rows.append(bias_1[t])
        for j in masters:
            group = (int(topk_idx[t, j]) // epr) if num_ranks < K else j
            key = (group, src_rank * max_tokens + t)
            rows.append(partial_of(key))
            if with_weights:
                wout[t] |= weights_of(key).numpy().view(np.uint32)
        out[t] = _ordered_sum_bf16(rows, hidden)
    return out, (None if wout is None else torch.from_numpy(wout.view(np.float32).copy()))


def rank_share_combine(y: torch.Tensor, expanded_weights: Optional[torch.Tensor], lay: dict, topk_idx: np.ndarray,
                       num_experts: int, max_tokens: int, bias_0=None, bias_1=None):
    """Single-rank (num_ranks == 1) dispatch->combine round trip: every partial is local."""
    parts, wv = combine_partial(y, expanded_weights, lay['recv_src_metadata'], 1, 0, max_tokens)
    H = y.shape[1]
    return combine_final(topk_idx, num_experts, 1, 0, max_tokens, lambda k: parts[k], lambda k: wv[k],
                         bias_0, bias_1, H, expanded_weights is not None)


def combine_fast(y: torch.Tensor, expanded_weights: Optional[torch.Tensor], meta: np.ndarray, num_tokens: int,
                 num_topk: int, bias_0=None, bias_1=None, rank_idx: int = 0, max_tokens: int = 0):
    """Vectorised num_ranks == 1 combine, identical in result to rank_share_combine; used at
    sizes where the per-token loops above would take minutes.  One master per token, so
    combined = BF16(sum_j f32 y[slot_j]) (verbatim for a single slot), then with biases
    BF16(f32 b0 + f32 b1 + f32 partial)."""
    N = meta.shape[0]
    K = num_topk
    H = y.shape[1]
    slots = torch.from_numpy(meta[:, :K].astype(np.int64))
    src = torch.from_numpy((meta[:, K].astype(np.int64) - rank_idx * max_tokens))
    valid = slots >= 0
    nvalid = valid.sum(dim=1)
    acc = torch.zeros((N, H), dtype=torch.float32)
    first = torch.zeros((N, H), dtype=torch.bfloat16)
    started = torch.zeros(N, dtype=torch.bool)
    for j in range(K):
        m = valid[:, j]
        take = m & ~started                          # the accumulator starts from the first row, not from +0
        cont = m & started
        first[take] = y[slots[take, j]]
        acc[take] = y[slots[take, j]].float()
        acc[cont] = acc[cont] + y[slots[cont, j]].float()
        started |= m
    partial = acc.to(torch.bfloat16)
    single = nvalid == 1
    partial[single] = first[single]
    out = torch.zeros((num_tokens, H), dtype=torch.bfloat16)
    out[src] = partial
    rows: List[torch.Tensor] = [b for b in (bias_0, bias_1) if b is not None]
    if rows:
        has = torch.zeros(num_tokens, dtype=torch.bool)
        has[src] = True
        acc2 = rows[0].float()
        for b in rows[1:]:
            acc2 = acc2 + b.float()
        res = torch.where(has.unsqueeze(1), acc2 + out.float(), acc2).to(torch.bfloat16)
        if len(rows) == 1:
            res[~has] = rows[0][~has]                 # one input -> verbatim copy
        out = res
    wout = None
    if expanded_weights is not None:
        wout = torch.zeros((num_tokens, K), dtype=torch.float32)
        wrow = torch.zeros((N, K), dtype=torch.float32)
        for j in range(K):
            m = valid[:, j]
            wrow[m, j] = expanded_weights[slots[m, j]]
        wout[src] = wrow
    return out, wout


def combine_weighted(y: torch.Tensor, expanded_weights: torch.Tensor, meta: np.ndarray, num_tokens: int,
                     num_topk: int, rank_idx: int = 0, max_tokens: int = 0) -> torch.Tensor:
    """Opt-in gate-weighted combine (not in the reference, whose expert GEMM applies the gate):
    combined[t] = BF16( sum_j f32(w_j) * f32(y[slot_j]) ), products and sums rounded separately
    in fp32, j ascending."""
    N = meta.shape[0]
    K = num_topk
    H = y.shape[1]
    slots = torch.from_numpy(meta[:, :K].astype(np.int64))
    src = torch.from_numpy((meta[:, K].astype(np.int64) - rank_idx * max_tokens))
    acc = torch.zeros((N, H), dtype=torch.float32)
    for j in range(K):
        m = slots[:, j] >= 0
        s = slots[m, j]
        acc[m] = acc[m] + expanded_weights[s].unsqueeze(1) * y[s].float()
    out = torch.zeros((num_tokens, H), dtype=torch.bfloat16)
    out[src] = acc.to(torch.bfloat16)
    return out
