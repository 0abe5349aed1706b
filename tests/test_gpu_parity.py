"""Parity of the HIP path (through the deep_ep API and the C ABI beneath it) against the CPU oracle,
on identical seeded inputs.  Integer / byte results are compared bit-exactly; BF16 combine results
are compared bit-exactly too (the oracle follows the same fp32 summation order), which is inside the
1e-2 abs / 1e-2 rel tolerance the path is specified to.
"""
import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_routing, make_tokens
from oracle import ep_oracle as O

pytestmark = pytest.mark.gpu

DEV = 'cuda'


def _deep_ep():
    import deep_ep
    return deep_ep


def _buffer(T, H, K, R=1, rank=0, fp8=False, **kw):
    de = _deep_ep()
    return de.EPBuffer(de.LocalGroup(rank, R), num_max_tokens_per_rank=T, hidden=H, num_topk=K,
                       use_fp8_dispatch=fp8, explicitly_destroy=True, **kw)


def _i32(t):
    return t.cpu().numpy().astype(np.int32)


def check_handle(handle, lay, do_cpu_sync=True):
    assert np.array_equal(_i32(handle.psum_num_recv_tokens_per_rank), lay['psum_num_recv_tokens_per_rank'])
    assert np.array_equal(_i32(handle.psum_num_recv_tokens_per_expert), lay['psum_num_recv_tokens_per_expert'])
    assert np.array_equal(_i32(handle.num_unaligned_recv_tokens_per_expert), lay['num_unaligned_recv_tokens_per_expert'])
    assert np.array_equal(_i32(handle.dst_buffer_slot_idx), lay['dst_buffer_slot_idx'])
    assert np.array_equal(_i32(handle.dst_gsge_idx), lay['dst_gsge_idx'])
    n = lay['num_recv_tokens']
    assert np.array_equal(_i32(handle.recv_src_metadata)[:n], lay['recv_src_metadata'])
    if do_cpu_sync:
        assert handle.num_recv_tokens == n
        assert handle.num_expanded_tokens == lay['num_expanded_tokens']
        assert handle.num_recv_tokens_per_expert_list == lay['num_recv_tokens_per_expert_list']
        assert handle.recv_src_metadata.size(0) == n


def valid_rows_mask(lay):
    m = np.zeros(lay['num_expanded_tokens'], dtype=bool)
    s = lay['recv_src_metadata'][:, :-2]
    m[s[s >= 0]] = True
    return m


CASES = [
    # T, H, E, K, A, masked, zipf
    (128, 256, 8, 2, 1, 0.0, None),        # reference's CPU-runnable shape
    (1, 256, 8, 2, 1, 0.0, None),
    (77, 512, 16, 4, 8, 0.2, None),
    (300, 1024, 64, 6, 128, 0.1, None),
    (128, 7168, 256, 8, 128, 0.1, 1.2),    # skewed decode-size routing: empty and hot experts
    (513, 2048, 32, 3, 16, 0.5, None),
    (64, 128, 2048, 32, 1, 0.0, None),     # the largest expert count and top-k the layout supports
]


@pytest.mark.parametrize('T,H,E,K,A,masked,zipf', CASES)
def test_bf16_dispatch_combine(T, H, E, K, A, masked, zipf):
    x = make_tokens(T, H, seed=T + H)
    topk, w = make_routing(T, E, K, seed=T, masked=masked, zipf=zipf)
    if T > 5:
        topk[3] = -1                      # a token nobody receives
        w[3] = 0
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    buf = _buffer(T, H, K)
    stats = torch.zeros(E, dtype=torch.int32, device=DEV)
    xg, tg, wg = x.to(DEV), topk.to(DEV), w.to(DEV)
    recv_x, recv_idx, recv_w, handle, ev = buf.dispatch(
        xg, topk_idx=tg, topk_weights=wg, cumulative_local_expert_recv_stats=stats, num_experts=E,
        num_max_tokens_per_rank=T, expert_alignment=A, do_expand=True, do_zero_padding=True, do_cpu_sync=True)
    torch.cuda.synchronize()
    assert recv_idx is None
    check_handle(handle, lay)
    assert np.array_equal(_i32(stats), lay['num_unaligned_recv_tokens_per_expert'])
    ex, _, ew = O.rank_share_dispatch(bf16_bits(x), None, w.numpy(), lay)
    assert np.array_equal(bf16_bits(recv_x), ex)                       # payload and zero padding, bitwise
    assert np.array_equal(recv_w.cpu().numpy().view(np.uint32), ew.view(np.uint32))

    # combine: expert outputs ~N(0,1) in every row (padding rows included, they must be ignored)
    g = torch.Generator().manual_seed(99)
    y = torch.randn((lay['num_expanded_tokens'], H), generator=g).to(torch.bfloat16)
    for nb in (0, 1, 2):
        bias = [torch.randn((T, H), generator=g).to(torch.bfloat16) for _ in range(nb)]
        b_arg = None if nb == 0 else (bias[0].to(DEV) if nb == 1 else tuple(b.to(DEV) for b in bias))
        cx, cw, _ = buf.combine(y.to(DEV), handle, topk_weights=recv_w, bias=b_arg)
        torch.cuda.synchronize()
        ox, ow = O.combine_fast(y, torch.from_numpy(ew), lay['recv_src_metadata'], T, K,
                                bias[0] if nb > 0 else None, bias[1] if nb > 1 else None)
        assert np.array_equal(bf16_bits(cx), bf16_bits(ox)), nb
        assert torch.equal(cw.cpu(), ow)
        assert torch.equal(cw.cpu(), w)                                 # weights make the round trip
    cx, cw, _ = buf.combine(y.to(DEV), handle)
    torch.cuda.synchronize()
    assert cw is None
    ox, _ = O.combine_fast(y, None, lay['recv_src_metadata'], T, K)
    assert np.array_equal(bf16_bits(cx), bf16_bits(ox))
    buf.destroy()


@pytest.mark.parametrize('T,H,E,K,A,masked,zipf', CASES[:6])
def test_fp8_dispatch_fused_and_prequantised(T, H, E, K, A, masked, zipf):
    de = _deep_ep()
    x = make_tokens(T, H, seed=T + H + 1, outliers=True)
    topk, w = make_routing(T, E, K, seed=T + 1, masked=masked, zipf=zipf)
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    q, s = O.quantise(x)
    eq, es, ew = O.rank_share_dispatch(q.numpy(), s.numpy().view(np.uint32), w.numpy(), lay)
    buf = _buffer(T, H, K, fp8=True)
    xg, tg, wg = x.to(DEV), topk.to(DEV), w.to(DEV)
    common = dict(num_experts=E, num_max_tokens_per_rank=T, expert_alignment=A, do_expand=True,
                  do_zero_padding=True)

    # fused quantise + scatter
    (rx, rsf), _, rw, handle, _ = buf.dispatch(xg, topk_idx=tg, topk_weights=wg, fused_fp8_quant=True, **common)
    torch.cuda.synchronize()
    check_handle(handle, lay)
    assert rx.dtype == torch.float8_e4m3fn and rsf.dtype == torch.float32
    assert np.array_equal(rx.view(torch.uint8).cpu().numpy(), eq)
    assert np.array_equal(rsf.cpu().numpy().view(np.uint32), es)
    assert np.array_equal(rw.cpu().numpy().view(np.uint32), ew.view(np.uint32))

    # the integer conversion path gives the same bytes
    de._C.set_fp8_hw_convert(False)
    try:
        (rx2, rsf2), _, _, _, _ = buf.dispatch(xg, topk_idx=tg, topk_weights=wg, fused_fp8_quant=True, **common)
        torch.cuda.synchronize()
    finally:
        de._C.set_fp8_hw_convert(True)
    assert torch.equal(rx2.view(torch.uint8), rx.view(torch.uint8)) and torch.equal(rsf2, rsf)

    # drop-in form: caller-side quantiser, scale packs viewed as int16, row- and column-major.  The helper gives
    # the oracle's bytes for a CPU tensor (torch's formula) and for a GPU tensor (the library's kernel) alike
    xq, xs = de.utils.math.per_token_cast_to_fp8(x)
    assert np.array_equal(xq.view(torch.uint8).numpy(), q.numpy())
    assert np.array_equal(xs.numpy().view(np.uint32), s.numpy().view(np.uint32))
    xq, xs = de.utils.math.per_token_cast_to_fp8(xg)
    assert xq.is_cuda and xq.dtype == torch.float8_e4m3fn and xs.dtype == torch.float32
    assert np.array_equal(xq.view(torch.uint8).cpu().numpy(), q.numpy())
    assert np.array_equal(xs.cpu().numpy().view(np.uint32), s.numpy().view(np.uint32))
    sf16 = xs.view(torch.int16)
    P = sf16.size(1)
    es16 = es.view(np.int16).reshape(es.shape[0], -1)
    for col_major in (False, True):
        if col_major:
            store = torch.empty((T * P,), dtype=torch.int16, device=DEV)
            sf_in = torch.as_strided(store, (T, P), (1, T))
            sf_in.copy_(sf16)
        else:
            sf_in = sf16
        (px, psf), _, pw, h2, _ = buf.dispatch((xq, sf_in), topk_idx=tg, topk_weights=wg,
                                               use_tma_aligned_col_major_sf=col_major, **common)
        torch.cuda.synchronize()
        check_handle(h2, lay)
        assert psf.stride() == ((1, px.size(0)) if col_major else (P, 1))
        assert np.array_equal(px.view(torch.uint8).cpu().numpy(), eq)
        assert np.array_equal(psf.cpu().numpy(), es16)
        assert np.array_equal(pw.cpu().numpy().view(np.uint32), ew.view(np.uint32))
    buf.destroy()


@pytest.mark.parametrize('R,rank', [(1, 0), (4, 2)])
@pytest.mark.parametrize('do_cpu_sync', [True, False])
def test_column_major_scales(R, rank, do_cpu_sync):
    """use_tma_aligned_col_major_sf: strides (1, N) exactly as the reference's transposing pass leaves
    them (tests/ep/test_ep.py:141-145), for fused and pre-quantised input, with and without the host
    sync, for a cached replay, and at R > 1 where fp32 scales travel as two 2-byte packs."""
    de = _deep_ep()
    T, H, E, K, A = 300, 1024, 16, 4, 32
    x = make_tokens(T, H, seed=9, outliers=True)
    topk, w = make_routing(T, E, K, seed=9, masked=0.2)
    lay = O.rank_share_layout(topk.numpy(), E, R, rank, A, T)
    q, s = O.quantise(x)
    eq, es, ew = O.rank_share_dispatch(q.numpy(), s.numpy().view(np.uint32), w.numpy(), lay)
    ne = lay['num_expanded_tokens']
    buf = _buffer(T, H, K, R=R, rank=rank, fp8=True)
    tg, wg = topk.to(DEV), w.to(DEV)
    common = dict(num_experts=E, num_max_tokens_per_rank=T, expert_alignment=A, do_expand=True,
                  do_zero_padding=True, do_cpu_sync=do_cpu_sync, use_tma_aligned_col_major_sf=True)

    def check(rx, rsf, expect_q, expect_s, view):
        n = rx.size(0)
        assert n == (ne if do_cpu_sync else O.no_sync_sizes(R, T, K, E, A)[1])
        assert rsf.shape == (n, expect_s.shape[1]) and rsf.stride() == (1, n)
        assert np.array_equal(rx.view(torch.uint8).cpu().numpy()[:ne], expect_q)
        assert np.array_equal(rsf.cpu().numpy().view(view)[:ne], expect_s)

    (rx, rsf), _, rw, handle, _ = buf.dispatch(x.to(DEV), topk_idx=tg, topk_weights=wg, fused_fp8_quant=True, **common)
    torch.cuda.synchronize()
    check(rx, rsf, eq, es, np.uint32)

    sf16 = s.view(torch.int16).to(DEV)
    es16 = es.view(np.int16).reshape(ne, -1)
    (px, psf), _, _, h2, _ = buf.dispatch((q.view(torch.float8_e4m3fn).to(DEV), sf16), topk_idx=tg, topk_weights=wg,
                                          **common)
    torch.cuda.synchronize()
    check(px, psf, eq, es16, np.int16)

    # cached replay with new payload
    x2 = make_tokens(T, H, seed=10)
    q2, s2 = O.quantise(x2)
    eq2, es2, _ = O.rank_share_dispatch(q2.numpy(), s2.numpy().view(np.uint32), w.numpy(), lay)
    (cx, csf), _, _, _, _ = buf.dispatch(x2.to(DEV), handle=handle, fused_fp8_quant=True, do_expand=True,
                                         do_zero_padding=True, use_tma_aligned_col_major_sf=True)
    torch.cuda.synchronize()
    check(cx, csf, eq2, es2, np.uint32)
    buf.destroy()


@pytest.mark.parametrize('packs', [3, 4, 66])
@pytest.mark.parametrize('alignment', [1, 2])
def test_column_major_two_byte_packs_of_any_shape(packs, alignment):
    """Pre-quantised input whose scale packs are any 2-byte type, asked for as columns: odd and even pack
    counts, odd and even row counts (the transposing kernel moves pairs of packs where both are even and
    single ones otherwise), more columns than one tile holds."""
    de = _deep_ep()
    T, H, E, K = 71, 128, 4, 2
    topk, w = make_routing(T, E, K, seed=3, masked=0.3)
    g = torch.Generator().manual_seed(packs)
    xq = torch.randint(0, 255, (T, H), generator=g, dtype=torch.uint8)
    sf = torch.randint(-32768, 32767, (T, packs), generator=g, dtype=torch.int16)
    seen = set()
    for drop in (0, 1):                     # one token less changes the parity of the row count at alignment 1
        tk = topk.clone()
        if drop:                            # token 0 gets one selection more or less than it had
            tk[0] = torch.tensor([0, -1] if int((topk[0] >= 0).sum()) != 1 else [0, 1])
        lay = O.rank_share_layout(tk.numpy(), E, 1, 0, alignment, T)
        ex, es, _ = O.rank_share_dispatch(xq.numpy(), sf.numpy().view(np.uint8).reshape(T, -1), w.numpy(), lay)
        buf = _buffer(T, H, K, fp8=True)
        (rx, rsf), _, _, handle, _ = buf.dispatch((xq.view(torch.float8_e4m3fn).to(DEV), sf.to(DEV)), topk_idx=tk.to(DEV),
                                                  topk_weights=w.to(DEV), num_experts=E, num_max_tokens_per_rank=T,
                                                  expert_alignment=alignment, do_expand=True, do_zero_padding=True,
                                                  use_tma_aligned_col_major_sf=True)
        torch.cuda.synchronize()
        n = lay['num_expanded_tokens']
        seen.add(n % 2)
        assert rsf.shape == (n, packs) and rsf.stride() == (1, n)
        assert np.array_equal(rx.view(torch.uint8).cpu().numpy(), ex)
        assert np.array_equal(rsf.cpu().numpy(), es.view(np.int16).reshape(n, packs))
        buf.destroy()
    if alignment == 1:
        assert seen == {0, 1}               # both parities of the row count were exercised


def test_fp8_hardware_conversion_matches_integer_conversion():
    """Every fp32 bit pattern with |x| <= 464 (the quantiser never exceeds 448*(1+2^-23))."""
    de = _deep_ep()
    bad, first = de._C.fp8_selftest(0, 1 << 32, 464.0)
    assert bad == 0, f'{bad} mismatches, first at bits {first:#x}'


def test_cached_dispatch_replays_layout():
    T, H, E, K, A = 200, 512, 32, 4, 16
    x = make_tokens(T, H, seed=5)
    topk, w = make_routing(T, E, K, seed=5, masked=0.15)
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    buf = _buffer(T, H, K)
    tg = topk.to(DEV)
    _, _, _, handle, _ = buf.dispatch(x.to(DEV), topk_idx=tg, topk_weights=w.to(DEV), num_experts=E,
                                      num_max_tokens_per_rank=T, expert_alignment=A, do_expand=True,
                                      do_zero_padding=True)
    torch.cuda.synchronize()
    saved = [t.clone() for t in (handle.psum_num_recv_tokens_per_rank, handle.psum_num_recv_tokens_per_expert,
                                 handle.num_unaligned_recv_tokens_per_expert, handle.recv_src_metadata,
                                 handle.dst_buffer_slot_idx, handle.dst_gsge_idx)]
    for send_weights in (True, False):
        x2 = make_tokens(T, H, seed=6 + send_weights) * (8 if send_weights else 0.125)
        w2 = torch.randn((T, K), generator=torch.Generator().manual_seed(8)).masked_fill(topk < 0, 0)
        rx, ridx, rw, h2, _ = buf.dispatch(x2.to(DEV), topk_weights=w2.to(DEV) if send_weights else None,
                                           handle=handle, do_expand=True, do_zero_padding=True,
                                           num_sms=0 if send_weights else handle.num_sms + 1)
        torch.cuda.synchronize()
        assert h2 is handle and ridx is None
        for t, s in zip((handle.psum_num_recv_tokens_per_rank, handle.psum_num_recv_tokens_per_expert,
                         handle.num_unaligned_recv_tokens_per_expert, handle.recv_src_metadata,
                         handle.dst_buffer_slot_idx, handle.dst_gsge_idx), saved):
            assert torch.equal(t, s)
        ex, _, ew = O.rank_share_dispatch(bf16_bits(x2), None, w2.numpy(), lay)
        assert np.array_equal(bf16_bits(rx), ex)
        if send_weights:
            assert np.array_equal(rw.cpu().numpy().view(np.uint32), ew.view(np.uint32))
        else:
            assert rw is None
    buf.destroy()


@pytest.mark.parametrize('unrouted', [(), (0,), (3, 77, 199)])
@pytest.mark.parametrize('do_cpu_sync', [True, False])
@pytest.mark.parametrize('fused', [False, True])
def test_cached_replay_whatever_rows_map_to_tokens(unrouted, do_cpu_sync, fused):
    """A cached replay fetches the payload of "row i = token i" ahead of the metadata row when the handle holds one
    metadata row per token, and fetches again when the row names another token.  Every token received (the guess is
    right), tokens nobody receives with exact counts (fewer rows than tokens: no guess), and the same with a handle of
    worst-case sizes (as many rows as tokens: the guess is wrong behind the first such token)."""
    T, H, E, K, A = 200, 512, 32, 4, 16
    topk, w = make_routing(T, E, K, seed=15)
    for t in unrouted:
        topk[t] = -1
        w[t] = 0
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    assert lay['num_recv_tokens'] == T - len(unrouted)
    buf = _buffer(T, H, K, fp8=fused)
    kw = dict(do_expand=True, do_zero_padding=True, fused_fp8_quant=fused)
    _, _, _, handle, _ = buf.dispatch(make_tokens(T, H, seed=1).to(DEV), topk_idx=topk.to(DEV), topk_weights=w.to(DEV),
                                      num_experts=E, num_max_tokens_per_rank=T, expert_alignment=A,
                                      do_cpu_sync=do_cpu_sync, **kw)
    assert handle.recv_src_metadata.size(0) == (lay['num_recv_tokens'] if do_cpu_sync else T)
    x2 = make_tokens(T, H, seed=2, outliers=True)
    recv, _, rw, _, _ = buf.dispatch(x2.to(DEV), topk_weights=w.to(DEV), handle=handle, **kw)
    torch.cuda.synchronize()
    ne = lay['num_expanded_tokens']
    if fused:
        q, sf = O.quantise(x2)
        ex, es, ew = O.rank_share_dispatch(q.numpy(), sf.numpy().view(np.uint32), w.numpy(), lay)
        assert np.array_equal(recv[0].view(torch.uint8).cpu().numpy()[:ne], ex)
        assert np.array_equal(recv[1].cpu().numpy().view(np.uint32)[:ne], es)
    else:
        ex, _, ew = O.rank_share_dispatch(bf16_bits(x2), None, w.numpy(), lay)
        assert np.array_equal(bf16_bits(recv)[:ne], ex)
    assert np.array_equal(rw.cpu().numpy().view(np.uint32)[:ne], ew.view(np.uint32))
    buf.destroy()


def test_dispatch_without_host_sync_uses_worst_case_sizes():
    T, H, E, K, A = 96, 256, 16, 4, 8
    x = make_tokens(T, H, seed=2)
    topk, w = make_routing(T, E, K, seed=2, masked=0.3)
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    buf = _buffer(T, H, K)
    rx, _, rw, handle, _ = buf.dispatch(x.to(DEV), topk_idx=topk.to(DEV), topk_weights=w.to(DEV), num_experts=E,
                                        num_max_tokens_per_rank=T, expert_alignment=A, do_expand=True,
                                        do_zero_padding=True, do_cpu_sync=False)
    torch.cuda.synchronize()
    n_recv, n_exp = O.no_sync_sizes(1, T, K, E, A)
    assert handle.num_recv_tokens == n_recv and handle.recv_src_metadata.size(0) == n_recv
    assert rx.size(0) == n_exp and handle.num_recv_tokens_per_expert_list == []
    check_handle(handle, lay, do_cpu_sync=False)
    ex, _, ew = O.rank_share_dispatch(bf16_bits(x), None, w.numpy(), lay)
    ne = lay['num_expanded_tokens']
    assert np.array_equal(bf16_bits(rx)[:ne], ex)
    y = make_tokens(n_exp, H, seed=3)
    cx, cw, _ = buf.combine(y.to(DEV), handle, topk_weights=rw)
    torch.cuda.synchronize()
    ox, ow = O.combine_fast(y, torch.from_numpy(ew), lay['recv_src_metadata'], T, K)
    assert np.array_equal(bf16_bits(cx), bf16_bits(ox))
    assert torch.equal(cw.cpu(), w)
    buf.destroy()


def test_weighted_combine_extension():
    T, H, E, K, A = 150, 512, 16, 4, 8
    topk, w = make_routing(T, E, K, seed=4, masked=0.2)
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    buf = _buffer(T, H, K)
    x = make_tokens(T, H, seed=4)
    _, _, rw, handle, _ = buf.dispatch(x.to(DEV), topk_idx=topk.to(DEV), topk_weights=w.to(DEV), num_experts=E,
                                       num_max_tokens_per_rank=T, expert_alignment=A, do_expand=True,
                                       do_zero_padding=True)
    y = make_tokens(lay['num_expanded_tokens'], H, seed=9)
    cx, _, _ = buf.combine(y.to(DEV), handle, topk_weights=rw, apply_weights=True)
    torch.cuda.synchronize()
    ox = O.combine_weighted(y, rw.cpu(), lay['recv_src_metadata'], T, K)
    assert np.array_equal(bf16_bits(cx), bf16_bits(ox))
    # and it is what a caller computes by hand: sum_j w_j y_j within tolerance
    ref = torch.zeros((T, H))
    meta = lay['recv_src_metadata']
    for i in range(meta.shape[0]):
        for j in range(K):
            if meta[i, j] >= 0:
                ref[meta[i, K]] += w[meta[i, K], j] * y[meta[i, j]].float()
    assert torch.allclose(cx.float().cpu(), ref, atol=1e-2, rtol=1e-2)
    buf.destroy()


def test_deferred_epilogue_and_event_hook():
    de = _deep_ep()
    T, H, E, K, A = 64, 1024, 8, 2, 4
    x = make_tokens(T, H, seed=12)
    topk, w = make_routing(T, E, K, seed=12)
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    buf = _buffer(T, H, K)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        xg = x.to(DEV)
        ev = buf.dispatch(xg, topk_idx=topk.to(DEV), topk_weights=w.to(DEV), num_experts=E,
                          num_max_tokens_per_rank=T, expert_alignment=A, do_expand=True, do_zero_padding=True,
                          async_with_compute_stream=True, defer_epilogue=True)
        assert isinstance(ev, de.EventOverlap)
        del xg                                     # the deferred epilogue must keep its input alive
        pressure = torch.full((T, H), -100, dtype=torch.bfloat16, device=DEV)
        rx, ridx, rw, handle = ev.current_stream_wait()
        assert ev.wait() is None                   # the hook runs once
        y = rx.clone()
        cev = buf.combine(y, handle, topk_weights=rw, async_with_compute_stream=True, defer_epilogue=True)
        cx, cw = cev.current_stream_wait(release_handle=True)
        assert cev.event is None
    stream.synchronize()
    del pressure
    ex, _, ew = O.rank_share_dispatch(bf16_bits(x), None, w.numpy(), lay)
    assert np.array_equal(bf16_bits(rx), ex)
    ox, _ = O.combine_fast(torch.from_numpy(ex.view(np.int16)).view(torch.bfloat16), None,
                           lay['recv_src_metadata'], T, K)
    assert np.array_equal(bf16_bits(cx), bf16_bits(ox))
    with pytest.raises(de._C.EPException):
        buf.dispatch(x.to(DEV), topk_idx=topk.to(DEV), num_experts=E, do_expand=True, defer_epilogue=True)
    buf.destroy()


def test_contract_violations_raise():
    de = _deep_ep()
    T, H, E, K = 32, 256, 8, 2
    buf = _buffer(T, H, K)
    x = make_tokens(T, H).to(DEV)
    topk, w = make_routing(T, E, K)
    kw = dict(num_experts=E, do_expand=True)
    with pytest.raises(de._C.EPException, match=r'Assertion exception \(ep_runtime.cpp:\d+\)'):
        buf.dispatch(x.float(), topk_idx=topk.to(DEV), **kw)                       # wrong dtype
    with pytest.raises(de._C.EPException, match='num_tokens <= a.num_max_tokens_per_rank'):
        buf.dispatch(torch.cat([x, x]), topk_idx=torch.cat([topk, topk]).to(DEV), **kw)
    with pytest.raises(de._C.EPException, match='EP_DTYPE_I64'):
        buf.dispatch(x, topk_idx=topk.to(DEV).int(), **kw)
    with pytest.raises(de._C.EPException, match='contiguous'):
        buf.dispatch(x.t().contiguous().t(), topk_idx=topk.to(DEV), **kw)
    with pytest.raises(AssertionError):
        buf.dispatch(x, topk_idx=topk.to(DEV), num_experts=E)                      # do_expand=False
    with pytest.raises(NotImplementedError):
        buf.dispatch(x, topk_idx=topk.to(DEV), num_qps=4, **kw)
    with pytest.raises(de._C.EPException, match='GPU'):
        buf.dispatch(x.cpu(), topk_idx=topk.to(DEV), **kw)
    buf.destroy()
    with pytest.raises(NotImplementedError):
        de.EPBuffer(de.LocalGroup(), num_bytes=0, sl_idx=1)
    with pytest.raises(de._C.EPException):
        de._C.calculate_ep_buffer_size(0, 1, 1, 1, False)


def test_host_count_wait_fails_at_once_without_host_sync():
    """A dispatch launched with do_cpu_sync=False never publishes the counts: waiting for them is a usage
    error and is reported at once, not after the CPU deadline."""
    import ctypes
    import time
    de = _deep_ep()
    T, H, E, K = 16, 128, 4, 2
    buf = _buffer(T, H, K, num_cpu_timeout_secs=100)
    topk, _ = make_routing(T, E, K)
    buf.dispatch(make_tokens(T, H).to(DEV), topk_idx=topk.to(DEV), num_experts=E, do_expand=True, do_cpu_sync=False)
    torch.cuda.synchronize()
    a, b = ctypes.c_int(), ctypes.c_int()
    t0 = time.perf_counter()
    rc = de._C._ep_wait(buf.runtime._h, ctypes.byref(a), ctypes.byref(b), None)
    assert rc != 0 and 'do_cpu_sync' in de._C._ep_last_error().decode()
    assert time.perf_counter() - t0 < 5
    buf.destroy()


def test_host_count_wait_times_out():
    """The counts do not arrive before the CPU deadline: the layout kernels sit behind about two seconds of
    other work on the stream (a bounded device-side spin that ends by itself), the buffer waits one second.
    The host gives up with the reference's "reduction timeout"; the stream then drains normally and the
    buffer is still good."""
    de = _deep_ep()
    T, H, E, K = 16, 128, 4, 2
    buf = _buffer(T, H, K, num_cpu_timeout_secs=1)
    topk, _ = make_routing(T, E, K)
    x, tk = make_tokens(T, H).to(DEV), topk.to(DEV)
    # cycles of the spin kernel per second, measured (its counter need not run at the shader clock)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda._sleep(1000)
    torch.cuda.synchronize()
    e0.record()
    torch.cuda._sleep(20_000_000)
    e1.record()
    torch.cuda.synchronize()
    cycles_per_sec = 20_000_000 / (e0.elapsed_time(e1) * 1e-3)
    assert 1e6 < cycles_per_sec < 1e11
    torch.cuda._sleep(int(2.0 * cycles_per_sec))
    with pytest.raises(de._C.EPException, match='reduction timeout'):
        buf.dispatch(x, topk_idx=tk, num_experts=E, do_expand=True, do_cpu_sync=True)
    torch.cuda.synchronize()
    _, _, _, handle, _ = buf.dispatch(x, topk_idx=tk, num_experts=E, do_expand=True, do_cpu_sync=True)
    torch.cuda.synchronize()
    assert handle.num_recv_tokens == T
    buf.destroy()


def test_lb_storage_aliases_arena_tail():
    de = _deep_ep()
    plan = de.BufferAllocator()
    weights = plan.allocate((4, 8), torch.float32)
    assert weights.is_meta
    buf = de.EPBuffer(de.LocalGroup(), num_bytes=de.get_num_allocation_alignment(),
                      lb_allocation_plan_or_num_bytes=plan, explicitly_destroy=True)
    assert weights.data_ptr() == buf.runtime.lb_storage.data_ptr()
    weights.fill_(3)
    torch.cuda.synchronize()
    assert (weights == 3).all()
    buf.destroy()


@pytest.mark.parametrize('T,H', [(1, 8), (33, 136), (7, 520), (64, 7168), (5, 16384)])
def test_gpu_quantiser_helper_matches_the_oracle(T, H):
    """deep_ep.utils.math.per_token_cast_to_fp8 on a GPU tensor runs the library's quantiser kernel: the oracle's
    bytes at every row length, also where the last group of 128 channels is short, with outliers and tiny rows."""
    g = torch.Generator().manual_seed(T * 1000 + H)
    x = torch.randn((T, H), generator=g)
    x[torch.rand((T, H), generator=g) < 0.01] *= 300
    x[0] *= 1e-6                                     # a row under the 1e-4 clamp
    x = x.to(torch.bfloat16)
    de = _deep_ep()
    q, s = O.quantise(x)
    xq, xs = de.utils.math.per_token_cast_to_fp8(x.to(DEV))
    torch.cuda.synchronize()
    assert xq.shape == (T, H) and xs.shape == (T, (H + 127) // 128)
    assert np.array_equal(xq.view(torch.uint8).cpu().numpy(), q.numpy())
    assert np.array_equal(xs.cpu().numpy().view(np.uint32), s.numpy().view(np.uint32))
    # a non-contiguous view goes through the torch formula on the tensor's own device (torch's GPU divisions round
    # differently from its CPU ones, so no bytes are compared): it still has to be a faithful quantisation
    wide = torch.randn((T, 2 * H), generator=g).to(torch.bfloat16).to(DEV)
    vq, vs = de.utils.math.per_token_cast_to_fp8(wide[:, :H])
    assert vq.shape == (T, H) and vs.shape == (T, (H + 127) // 128)
    back = de.utils.math.per_token_cast_back(vq, vs).float()
    ref = wide[:, :H].float()
    assert ((back - ref).abs() <= 0.07 * ref.abs().amax(dim=1, keepdim=True) + 1e-6).all()
