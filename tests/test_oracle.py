"""Pins the CPU oracle (oracle/ep_oracle.py) before anything is compared against it.

Evidence used, per function:
  * golden vectors written from the reference's own math.py / refs.py (tests/golden/*.npz);
  * the two-rank worked example derived by hand from the reference kernels;
  * a sequential, per-core simulation of the reference kernels (written independently of the
    oracle's vectorised closed forms) on random tiny inputs;
  * closed forms and exact special cases.
"""
import os

import numpy as np
import pytest
import torch

from helpers import bf16_from_bits, make_routing, make_tokens
from oracle import ep_oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')


# ---------------------------------------------------------------------------------------
# token layout byte counts (layout/ep/token.hpp:24-45)
# ---------------------------------------------------------------------------------------
def test_token_layout_sizes():
    assert O.dispatch_token_layout(7168, 112, 6).num_bytes() == 7488
    assert O.dispatch_token_layout(14336, 0, 6).num_bytes() == 14432
    assert O.dispatch_token_layout(14336, 0, 8).num_bytes() == 14464
    assert O.dispatch_token_layout(7168, 112, 8).num_bytes() == 7520
    assert O.combine_token_layout(7168, 6).num_bytes() == 14368
    assert O.combine_token_layout(7168, 8).num_bytes() == 14368
    lay = O.dispatch_token_layout(7168, 112, 6)
    assert (lay.sf_offset, lay.topk_idx_offset, lay.topk_weights_offset, lay.src_token_global_idx_offset) == \
        (7168, 7392, 7456, 7480)
    # cached mode: only the K weights travel
    assert O.dispatch_token_layout(14336, 0, 6, cached=True).num_bytes() == 14336 + 32


def test_buffer_size_hint():
    # max(dispatch, combine) aligned to 2 MiB; K=0 reserves 32 slots
    assert O.calculate_buffer_size(1, 16384, 7168, 6, False) == 236978176
    assert O.calculate_buffer_size(1, 16384, 7168, 6, True) == 236978176
    k0 = O.calculate_buffer_size(2, 128, 256, 0, False)
    assert k0 % O.ALLOC_ALIGN == 0 and k0 >= 2 * 128 * (512 + 128 + 256 + 32)


# ---------------------------------------------------------------------------------------
# quantiser
# ---------------------------------------------------------------------------------------
def test_quantise_golden():
    g = np.load(os.path.join(GOLD, 'quant_golden.npz'))
    names = sorted({k.rsplit('.', 1)[0] for k in g.files})
    assert len(names) == 4
    for n in names:
        x = bf16_from_bits(g[n + '.x'])
        q, s = O.quantise(x)
        assert np.array_equal(q.numpy(), g[n + '.q']), n
        assert np.array_equal(s.numpy().view(np.uint32), g[n + '.s'].view(np.uint32)), n


def _e4m3fn_encode_int(f: np.ndarray) -> np.ndarray:
    """Independent integer implementation of fp32 -> e4m3fn (RNE, no saturation, >464 -> NaN)."""
    bits = f.astype(np.float32).view(np.uint32).astype(np.uint64)
    sign = ((bits >> 24) & 0x80).astype(np.uint8)
    a = bits & 0x7FFFFFFF
    out = np.zeros(f.shape, dtype=np.uint8)
    exp = (a >> 23).astype(np.int64) - 127
    man = (a & 0x7FFFFF) | 0x800000
    # normal e4m3 range: unbiased exponent >= -6; below, the value is rounded to a multiple of 2^-9
    shift = np.where(exp >= -6, 20, 20 + (-6 - exp))
    shift = np.minimum(shift, 40)
    m64 = man.astype(np.uint64)
    q = m64 >> shift.astype(np.uint64)
    rem = m64 & ((np.uint64(1) << shift.astype(np.uint64)) - np.uint64(1))
    half = np.uint64(1) << (shift.astype(np.uint64) - np.uint64(1))
    up = (rem > half) | ((rem == half) & ((q & np.uint64(1)) == 1))
    q = q + up.astype(np.uint64)
    # normal: q has the hidden bit at position 3 -> code = (exp+7)<<3 | (q-8), carries propagate naturally
    code_norm = ((exp + 7) << 3) + (q.astype(np.int64) - 8)
    code_sub = q.astype(np.int64)
    code = np.where(exp >= -6, code_norm, code_sub)
    code = np.where(code > 0x7E, 0x7F, code)
    code = np.where(a > 0x7F800000, 0x7F, code)          # NaN
    code = np.where(a == 0, 0, code)
    out = (code.astype(np.uint8) | sign)
    return out


def test_e4m3fn_rounding_matches_independent_encoder():
    # every BF16 value, widened to fp32, times a handful of scales
    all_bf16 = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    np.seterr(all='ignore')
    for scale in (1.0, 448.0 / 3.0, 448.0 / 0.0123, 2.0 ** -7, 448.0 / 1e-4):
        f = (all_bf16 * np.float32(scale)).astype(np.float32)
        t = torch.from_numpy(f.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        mine = _e4m3fn_encode_int(f)
        finite = np.isfinite(f)
        assert np.array_equal(t[finite], mine[finite]), scale
    # boundary cases spelled out
    f = np.array([448., 449., 463.99, 464.0, 464.1, -448., 2.0 ** -9, 2.0 ** -10, 2.0 ** -10 * 1.0001, 0.0],
                 dtype=np.float32)
    exp = np.array([0x7E, 0x7E, 0x7E, 0x7E, 0x7F, 0xFE, 0x01, 0x00, 0x01, 0x00], dtype=np.uint8)
    assert np.array_equal(_e4m3fn_encode_int(f), exp)
    assert np.array_equal(torch.from_numpy(f).to(torch.float8_e4m3fn).view(torch.uint8).numpy(), exp)


def test_quantise_closed_forms():
    # all-zero group: scale = 1e-4/448, payload zero
    x = torch.zeros((2, 256), dtype=torch.bfloat16)
    # group with amax = 448 * 2^n: scale = 2^n exactly and payload = e4m3 encoding of x / 2^n
    x[1, 0] = 448.0 * 4
    x[1, 1] = -448.0 * 4
    x[1, 2] = 1.5 * 4        # 1.5 = 0x3C
    x[1, 3] = 2.0 ** -6 * 4  # smallest normal 0x08
    x[1, 4] = 2.0 ** -9 * 4  # smallest subnormal 0x01
    q, s = O.quantise(x)
    assert torch.all(q[0] == 0)
    assert s[0, 0].item() == np.float32(np.float32(1e-4) / np.float32(448.0))
    assert s[1, 0].item() == 4.0
    assert q[1, :5].tolist() == [0x7E, 0xFE, 0x3C, 0x08, 0x01]
    assert s[1, 1].item() == np.float32(np.float32(1e-4) / np.float32(448.0))
    # the multiplier is fl(fl(1/amax) * 448), two roundings (torch's `448.0 / tensor`), not one division
    am = np.float32(1.046875)
    two_step = np.float32(np.float32(1) / am) * np.float32(448)
    assert two_step != np.float32(448) / am
    xs = torch.zeros((1, 128), dtype=torch.bfloat16)
    xs[0, 0] = float(am)
    xs[0, 1:] = torch.linspace(0.01, 1.04, 127).to(torch.bfloat16)
    qs, _ = O.quantise(xs)
    want = torch.from_numpy((xs.float().numpy() * two_step).astype(np.float32)).to(torch.float8_e4m3fn).view(torch.uint8)
    assert torch.equal(qs, want)
    # multiply-by-reciprocal, not divide-by-scale
    g = torch.Generator().manual_seed(5)
    xx = (torch.randn((64, 128), generator=g) * 7).to(torch.bfloat16)
    q, s = O.quantise(xx)
    amax = xx.float().abs().amax(dim=1, keepdim=True)
    via_mul = (xx.float() * (448.0 / amax)).to(torch.float8_e4m3fn).view(torch.uint8)
    assert torch.equal(q, via_mul)


# ---------------------------------------------------------------------------------------
# worked two-rank example (derived by hand from the reference kernels)
# ---------------------------------------------------------------------------------------
def test_worked_micro_example():
    R, E, K, A, maxT = 2, 4, 2, 2, 4
    topk = np.array([[0, 1], [3, -1], [2, 0]], dtype=np.int64)
    dst, cnt, hist = O.send_layout(topk, E, R)
    assert dst.tolist() == [[-1, 0], [0, -1], [1, 1]]
    assert cnt.tolist() == [2, 2]
    assert hist.tolist() == [2, 1, 1, 1]
    lay = O.rank_share_layout(topk, E, R, 0, A, maxT)
    assert lay['psum_num_recv_tokens_per_rank'].tolist() == [2, 2]
    assert lay['num_unaligned_recv_tokens_per_expert'].tolist() == [2, 1]
    assert lay['psum_num_recv_tokens_per_expert'].tolist() == [2, 3]
    assert lay['num_expanded_tokens'] == 4
    assert lay['num_recv_tokens_per_expert_list'] == [2, 2]
    assert lay['recv_src_metadata'].tolist() == [[0, 2, 0, 1], [-1, 1, 2, 1]]
    x = np.arange(3 * 4, dtype=np.uint8).reshape(3, 4) + 1
    w = np.array([[.1, .2], [.3, 0], [.4, .5]], dtype=np.float32)
    rx, _, rw = O.rank_share_dispatch(x, None, w, lay)
    assert rx.tolist() == [x[0].tolist(), x[2].tolist(), x[0].tolist(), [0, 0, 0, 0]]
    assert rw.tolist() == [w[0, 0], w[2, 1], w[0, 1], 0.0]


# ---------------------------------------------------------------------------------------
# sequential simulation of the reference kernels, independent of the vectorised oracle
# ---------------------------------------------------------------------------------------
def _simulate(topk, E, R, rank_idx, A, maxT, num_cores=3):
    """Per-core, per-token walk as the device code does it (impls/ep/dispatch.hpp:166-292 for the
    send side with in-order arrival, dispatch_copy_epilogue.hpp:280-283,397-429,459-522 for the
    receive side)."""
    T, K = len(topk), len(topk[0])
    epr = E // R
    per_core = -(-T // num_cores)
    rank_fill = [0] * R
    dst = [[-1] * K for _ in range(T)]
    for c in range(num_cores):
        for t in range(c * per_core, min(T, (c + 1) * per_core)):
            for j in range(K):
                e = topk[t][j]
                if e < 0:
                    continue
                r = e // epr
                later = any(topk[t][jj] >= 0 and topk[t][jj] // epr == r for jj in range(j + 1, K))
                if not later:
                    dst[t][j] = rank_fill[r]
                    rank_fill[r] += 1
    # region of this rank: tokens in slot order
    region = [None] * rank_fill[rank_idx]
    for t in range(T):
        for j in range(K):
            if dst[t][j] >= 0 and topk[t][j] // epr == rank_idx:
                region[dst[t][j]] = t
    cnt = [0] * epr
    for t in region:
        for j in range(K):
            le = topk[t][j] - rank_idx * epr
            if topk[t][j] >= 0 and 0 <= le < epr:
                cnt[le] += 1
    start, psum, acc = [], [], 0
    for e in range(epr):
        start.append(acc)
        psum.append(acc + cnt[e])
        acc += -(-cnt[e] // A) * A
    nxt = list(start)
    meta = []
    for t in region:
        row, master = [], -1
        for j in range(K):
            le = topk[t][j] - rank_idx * epr
            if topk[t][j] >= 0 and 0 <= le < epr:
                row.append(nxt[le])
                nxt[le] += 1
                master = j
            else:
                row.append(-1)
        meta.append(row + [rank_idx * maxT + t, master])
    return dst, rank_fill, cnt, psum, meta, acc


@pytest.mark.parametrize('seed', range(12))
def test_layout_matches_sequential_simulation(seed):
    rng = np.random.default_rng(seed)
    R = int(rng.choice([1, 2, 4]))
    epr = int(rng.choice([1, 2, 3, 8]))
    E = R * epr
    K = int(rng.integers(1, min(E, 5) + 1))
    T = int(rng.integers(1, 40))
    A = int(rng.choice([1, 2, 8]))
    rank_idx = int(rng.integers(0, R))
    maxT = T + int(rng.integers(0, 5))
    topk = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int64)
    topk[rng.random((T, K)) < 0.25] = -1
    if seed % 3 == 0 and K > 1:                      # duplicates of the same expert are legal input
        topk[:, 1] = topk[:, 0]
    dst, fill, cnt, psum, meta, nexp = _simulate(topk.tolist(), E, R, rank_idx, A, maxT)
    lay = O.rank_share_layout(topk, E, R, rank_idx, A, maxT)
    assert lay['dst_buffer_slot_idx'].tolist() == dst
    assert lay['num_send_tokens_per_rank'].tolist() == fill
    assert lay['num_unaligned_recv_tokens_per_expert'].tolist() == cnt
    assert lay['psum_num_recv_tokens_per_expert'].tolist() == psum
    assert lay['recv_src_metadata'].tolist() == meta
    assert lay['num_expanded_tokens'] == nexp
    assert lay['psum_num_recv_tokens_per_rank'].tolist() == [0 if r < rank_idx else fill[rank_idx] for r in range(R)]


def test_layout_invariants_reference_test_asserts():
    """The invariants of tests/ep/test_ep.py:199-208,252-296 on a mid-size random case."""
    T, E, K, A = 512, 64, 6, 16
    topk, w = make_routing(T, E, K, seed=3, masked=0.1)
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    meta = lay['recv_src_metadata']
    slots = meta[:, :K]
    valid = slots >= 0
    recv_tok = meta[:, K]
    assert np.array_equal(valid, topk.numpy()[recv_tok] >= 0)
    v = slots[valid]
    assert v.size == lay['num_unaligned_recv_tokens_per_expert'].sum()
    assert np.unique(v).size == v.size and v.max() < lay['num_expanded_tokens']
    ps = [0] + lay['psum_num_recv_tokens_per_expert'].tolist()
    for e in range(E):
        s0 = O.align(ps[e], A)
        es = np.sort(slots[topk.numpy()[recv_tok] == e])
        assert np.array_equal(es, np.arange(s0, ps[e + 1]))
    master = np.where(valid, np.arange(K)[None], -1).max(axis=1)
    assert np.array_equal(meta[:, K + 1], master)
    # deterministic order: inside an expert, slots ascend with the source token
    for e in range(E):
        tt, jj = np.nonzero(topk.numpy()[recv_tok] == e)
        assert np.all(np.diff(slots[tt, jj]) > 0)


# ---------------------------------------------------------------------------------------
# dispatch ordering / masking against refs.dispatch run under a 2-rank gloo group
# ---------------------------------------------------------------------------------------
def test_dispatch_golden_two_ranks():
    g = np.load(os.path.join(GOLD, 'dispatch_golden_w2.npz'))
    W = 2
    ins = []
    for r in range(W):
        T, K, E, H, maxT, world = g[f'r{r}.cfg'].tolist()
        assert world == W
        ins.append((g[f'r{r}.x'], g[f'r{r}.topk_idx'], g[f'r{r}.topk_weights']))
    # every source packs its regions
    regions = []
    for s, (xb, idx, w) in enumerate(ins):
        dst, cnt, _ = O.send_layout(idx, E, W)
        regions.append(O.pack_regions(xb.view(np.uint8).reshape(xb.shape[0], -1), None, idx, w, dst, cnt,
                                      E, W, s, maxT))
    lay = O.dispatch_token_layout(H * 2, 0, K)
    for d in range(W):
        stream = np.concatenate([regions[s][d] for s in range(W)], axis=0)
        counts = [regions[s][d].shape[0] for s in range(W)]
        assert counts == g[f'r{d}.num_recv_tokens_per_rank'].tolist()
        hidden = stream[:, :H * 2].copy().view(np.uint16)
        assert np.array_equal(hidden, g[f'r{d}.recv_x'])
        idx = stream[:, lay.topk_idx_offset:lay.topk_idx_offset + 8 * K].copy().view(np.int64)
        w = stream[:, lay.topk_weights_offset:lay.topk_weights_offset + 4 * K].copy().view(np.float32)
        src = stream[:, lay.src_token_global_idx_offset:lay.src_token_global_idx_offset + 4].copy().view(np.int32)[:, 0]
        assert np.array_equal(src, g[f'r{d}.recv_src_token_idx'])
        assert np.array_equal(w, g[f'r{d}.recv_topk_weights'])
        epr = E // W
        local = np.where((idx >= d * epr) & (idx < (d + 1) * epr), idx - d * epr, -1)
        assert np.array_equal(local, g[f'r{d}.recv_topk_idx'])
        # and the expanded layout obeys the golden's per-expert counts
        rl = O.recv_layout(idx, src, counts, E, W, d, 4)
        for e in range(epr):
            assert rl['num_unaligned_recv_tokens_per_expert'][e] == (g[f'r{d}.recv_topk_idx'] == e).sum()


# ---------------------------------------------------------------------------------------
# combine against refs.combine(reduce_in_local=True) run under gloo groups of 1, 2 and 4 ranks
# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize('world', [1, 2, 4])
def test_combine_golden(world):
    g = np.load(os.path.join(GOLD, f'combine_golden_w{world}.npz'))
    ncases = len({k.split('.')[1] for k in g.files})
    assert ncases == 5
    for ci in range(ncases):
        p = f'w{world}.c{ci}.'
        T, K, E, H, nbias, W = g[p + 'cfg'].tolist()
        y = bf16_from_bits(g[p + 'y'])                       # [T,K,H] expert outputs per (t, j)
        topk = g[p + 'topk_idx']
        bias = [bf16_from_bits(g[p + f'bias{b}']) for b in range(nbias)]
        yflat = y.reshape(T * K, H)
        maxT = T
        epr = E // W
        parts, wvecs = {}, {}
        ew = torch.arange(T * K, dtype=torch.float32) + 1    # weight of slot s = s+1, to check the OR-merge
        for r in range(W):
            hits = ((topk >= r * epr) & (topk < (r + 1) * epr)).any(axis=1)
            toks = np.nonzero(hits)[0]
            meta = np.full((len(toks), K + 2), -1, dtype=np.int32)
            for i, t in enumerate(toks):
                for j in range(K):
                    if topk[t, j] >= 0 and topk[t, j] // epr == r:
                        meta[i, j] = t * K + j
                        meta[i, K + 1] = j
                meta[i, K] = t                                  # source rank 0
            pr, wv = O.combine_partial(yflat, ew, meta, W, r, maxT)
            assert not (set(pr) & set(parts))
            parts.update(pr)
            wvecs.update(wv)
        out, wout = O.combine_final(topk, E, W, 0, maxT, lambda k: parts[k], lambda k: wvecs[k],
                                    bias[0] if nbias > 0 else None, bias[1] if nbias > 1 else None, H, True)
        # the reference zeroes masked y and adds exact zeros, so only the sign of zero may differ
        assert torch.equal(out, bf16_from_bits(g[p + 'out'])), (world, ci)
        exp_w = np.where(topk >= 0, (np.arange(T * K).reshape(T, K) + 1).astype(np.float32), 0)
        assert np.array_equal(wout.numpy(), exp_w)


def test_combine_fast_equals_two_phase():
    T, E, K, H, A = 96, 16, 4, 64, 8
    topk, w = make_routing(T, E, K, seed=11, masked=0.3)
    topk[5] = -1                                              # a token nobody receives
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    g = torch.Generator().manual_seed(3)
    y = torch.randn((lay['num_expanded_tokens'], H), generator=g).to(torch.bfloat16)
    ew = torch.rand(lay['num_expanded_tokens'], generator=g)
    for nb in (0, 1, 2):
        b = [torch.randn((T, H), generator=g).to(torch.bfloat16) for _ in range(nb)]
        b0 = b[0] if nb > 0 else None
        b1 = b[1] if nb > 1 else None
        slow, wslow = O.rank_share_combine(y, ew, lay, topk.numpy(), E, T, b0, b1)
        fast, wfast = O.combine_fast(y, ew, lay['recv_src_metadata'], T, K, b0, b1)
        assert torch.equal(slow.view(torch.int16), fast.view(torch.int16)), nb
        assert torch.equal(wslow, wfast)


def test_combine_exact_cases():
    # K = 1: identity copy; equal powers of two: exact sums
    T, E, H = 8, 4, 16
    topk = torch.arange(T).remainder(E).view(T, 1).to(torch.int64)
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, 1, T)
    y = make_tokens(lay['num_expanded_tokens'], H, seed=1)
    out, _ = O.combine_fast(y, None, lay['recv_src_metadata'], T, 1)
    slots = lay['recv_src_metadata'][:, 0]
    assert torch.equal(out, y[torch.from_numpy(slots.astype(np.int64))])
    topk = torch.tensor([[0, 1, 2, 3]] * 4, dtype=torch.int64)
    lay = O.rank_share_layout(topk.numpy(), 4, 1, 0, 1, 4)
    y = torch.full((16, H), 0.25, dtype=torch.bfloat16)
    out, _ = O.combine_fast(y, None, lay['recv_src_metadata'], 4, 4)
    assert torch.all(out == 1.0)


# ---------------------------------------------------------------------------------------
# output sizes without a host sync (csrc/buffers/ep.hpp:288,316-320)
# ---------------------------------------------------------------------------------------
def test_no_sync_sizes_literals():
    # headline shape, one partition: 16384 * min(6, 256) + 127 * 256 = 130 816 rows, a multiple of 128
    assert O.no_sync_sizes(1, 16384, 6, 256, 128) == (16384, 130816)
    # 32 partitions of 8 experts: 32 * 16384 * min(6, 8) + 127 * 8 = 3 146 744 -> next multiple of 128
    assert O.no_sync_sizes(32, 16384, 6, 256, 128) == (524288, 3146752)
    # by hand: R=2, maxT=4, K=2, E=4 (2 experts a partition), A=2 -> 2*4*min(2,2) + (2-1)*2 = 18
    assert O.no_sync_sizes(2, 4, 2, 4, 2) == (8, 18)
    # top-k larger than the local experts: a row has at most one slot per local expert
    assert O.no_sync_sizes(4, 10, 8, 8, 1) == (40, 4 * 10 * 2)
    # alignment rounding of the total: 1*3*1 + 4*1 = 7 -> 10
    assert O.no_sync_sizes(1, 3, 1, 1, 5) == (3, 10)


def test_no_sync_sizes_bound_every_layout():
    # the bound holds for, and is reached by, the layouts it sizes: brute force over tiny routings
    rng = np.random.default_rng(0)
    for _ in range(200):
        R = int(rng.integers(1, 4))
        El = int(rng.integers(1, 4))
        E, K, A, T = R * El, int(rng.integers(1, 5)), int(rng.integers(1, 6)), int(rng.integers(1, 7))
        K = min(K, E)
        topk = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int64)
        topk[rng.random((T, K)) < 0.2] = -1
        n_recv_bound, n_exp_bound = O.no_sync_sizes(R, T, K, E, A)
        assert n_recv_bound == R * T and n_exp_bound % A == 0
        for r in range(R):
            lay = O.rank_share_layout(topk, E, R, r, A, T)
            # a single sender delivers at most T rows and T * min(K, El) slots
            assert lay['num_recv_tokens'] <= T
            assert lay['num_expanded_tokens'] <= n_exp_bound
    # worst case: every partition sends every token to all local experts, counts are 1 mod A
    R, El, K, A, T = 2, 2, 2, 4, 5
    cnt = R * T                                  # rows per local expert
    assert El * O.align(cnt, A) <= O.no_sync_sizes(R, T, K, R * El, A)[1]


# ---------------------------------------------------------------------------------------
# gate-weighted combine (extension): sum_j w_j * y_j in fp32, j ascending, one rounding
# ---------------------------------------------------------------------------------------
def test_combine_weighted_brute_force():
    T, E, K, H, A = 40, 8, 3, 24, 4
    topk, _ = make_routing(T, E, K, seed=5, masked=0.25)
    topk[7] = -1
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    g = torch.Generator().manual_seed(9)
    n_exp = lay['num_expanded_tokens']
    y = torch.randn((n_exp, H), generator=g).to(torch.bfloat16)
    ew = torch.rand(n_exp, generator=g)
    got = O.combine_weighted(y, ew, lay['recv_src_metadata'], T, K)
    # independent per-element loop in numpy float32: the expanded slot of (t, j) from the closed form
    # slot(t,j) = start[e] + #{earlier (t',j') with the same expert}
    tk = topk.numpy()
    cnt = np.zeros(E, np.int64)
    for t in range(T):
        for j in range(K):
            if tk[t, j] >= 0:
                cnt[tk[t, j]] += 1
    start = np.zeros(E, np.int64)
    for e in range(1, E):
        start[e] = start[e - 1] + (cnt[e - 1] + A - 1) // A * A
    fill = np.zeros(E, np.int64)
    yf = y.float().numpy()
    wf = ew.numpy()
    exp = np.zeros((T, H), np.float32)
    for t in range(T):
        for j in range(K):
            e = tk[t, j]
            if e < 0:
                continue
            s = start[e] + fill[e]
            fill[e] += 1
            for h in range(H):
                exp[t, h] = np.float32(exp[t, h] + np.float32(wf[s] * yf[s, h]))
    exp_bf = torch.from_numpy(exp).to(torch.bfloat16)
    assert torch.equal(got.view(torch.int16), exp_bf.view(torch.int16))
    # all weights 1 -> the plain combine (more than one slot: same sum, same rounding)
    ones = torch.ones(n_exp)
    plain, _ = O.combine_fast(y, None, lay['recv_src_metadata'], T, K)
    assert torch.equal(O.combine_weighted(y, ones, lay['recv_src_metadata'], T, K).view(torch.int16),
                       plain.view(torch.int16))
