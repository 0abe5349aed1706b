"""The benchmark configurations at full size: oracle comparison where the oracle finishes in seconds,
plus size-independent properties (permutation, zero padding, determinism, count identities)."""
import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_routing, make_tokens
from oracle import ep_oracle as O

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def _buffer(T, H, K, R=1, rank=0, fp8=False):
    import deep_ep
    return deep_ep.EPBuffer(deep_ep.LocalGroup(rank, R), num_max_tokens_per_rank=T, hidden=H, num_topk=K,
                            use_fp8_dispatch=fp8, explicitly_destroy=True)


def _check_layout_properties(handle, topk_dev, E, A, recv_rows, src_rows):
    """recv_rows[slot(t,j)] == src_rows[t] for every valid (t,j); padding rows are zero; slots are a
    permutation of the per-expert ranges (tests/ep/test_ep.py:199-221,280-296)."""
    meta = handle.recv_src_metadata.long()
    K = meta.size(1) - 2
    slots, src = meta[:, :K], meta[:, K]
    valid = slots >= 0
    assert torch.equal(valid, topk_dev[src] >= 0)
    vs = slots[valid]
    assert vs.numel() == int(handle.num_unaligned_recv_tokens_per_expert.sum())
    assert torch.unique(vs).numel() == vs.numel()
    expect = src_rows[src].unsqueeze(1).expand(-1, K, -1)[valid]
    assert torch.equal(recv_rows[vs], expect)
    pad = torch.ones(recv_rows.size(0), dtype=torch.bool, device=DEV)
    pad[vs] = False
    assert int(recv_rows[pad].count_nonzero()) == 0
    ps = handle.psum_num_recv_tokens_per_expert.long()
    cnt = handle.num_unaligned_recv_tokens_per_expert.long()
    start = ps - cnt
    assert torch.all(start % A == 0)
    assert torch.equal(cnt, torch.bincount(topk_dev[topk_dev >= 0], minlength=E))
    master = torch.where(valid, torch.arange(K, device=DEV).view(1, K), torch.full_like(slots, -1)).max(dim=1).values
    assert torch.equal(meta[:, K + 1], master)


def test_c2_bf16_top8_full_oracle():
    T, H, E, K, A = 4096, 7168, 256, 8, 128
    x = make_tokens(T, H, seed=0, outliers=True)
    topk, w = make_routing(T, E, K, seed=0)
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    buf = _buffer(T, H, K)
    rx, _, rw, handle, _ = buf.dispatch(x.to(DEV), topk_idx=topk.to(DEV), topk_weights=w.to(DEV), num_experts=E,
                                        expert_alignment=A, do_expand=True, do_zero_padding=True)
    torch.cuda.synchronize()
    assert np.array_equal(handle.recv_src_metadata.cpu().numpy(), lay['recv_src_metadata'])
    ex, _, ew = O.rank_share_dispatch(bf16_bits(x), None, w.numpy(), lay)
    assert np.array_equal(bf16_bits(rx), ex)
    assert np.array_equal(rw.cpu().numpy().view(np.uint32), ew.view(np.uint32))
    y = torch.randn((rx.size(0), H), generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    cx, cw, _ = buf.combine(y.to(DEV), handle, topk_weights=rw)
    torch.cuda.synchronize()
    ox, ow = O.combine_fast(y, torch.from_numpy(ew), lay['recv_src_metadata'], T, K)
    assert np.array_equal(bf16_bits(cx), bf16_bits(ox))
    assert (cx.float().cpu() - ox.float()).abs().max() <= 1e-2        # the stated tolerance, trivially
    assert torch.equal(cw.cpu(), w)
    buf.destroy()


def test_c3_headline_fp8_dispatch_bf16_combine():
    T, H, E, K, A = 16384, 7168, 256, 6, 128
    x = make_tokens(T, H, seed=0, outliers=True)
    topk, w = make_routing(T, E, K, seed=0)
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    q, s = O.quantise(x)
    buf = _buffer(T, H, K, fp8=True)
    xg, tg, wg = x.to(DEV), topk.to(DEV), w.to(DEV)
    kw = dict(num_experts=E, expert_alignment=A, do_expand=True, do_zero_padding=True, fused_fp8_quant=True)
    (rx, rsf), _, rw, handle, _ = buf.dispatch(xg, topk_idx=tg, topk_weights=wg, **kw)
    torch.cuda.synchronize()
    assert handle.num_expanded_tokens == lay['num_expanded_tokens'] == rx.size(0)
    assert np.array_equal(handle.recv_src_metadata.cpu().numpy(), lay['recv_src_metadata'])
    assert np.array_equal(handle.psum_num_recv_tokens_per_expert.cpu().numpy(), lay['psum_num_recv_tokens_per_expert'])
    # payload and scales: every valid slot holds the oracle's quantised row, padding is zero
    _check_layout_properties(handle, tg, E, A, rx.view(torch.uint8), q.to(DEV))
    _check_layout_properties(handle, tg, E, A, rsf.view(torch.int32), s.view(torch.int32).to(DEV))
    ex, es, ew = O.rank_share_dispatch(q.numpy(), s.numpy().view(np.uint32), w.numpy(), lay)
    assert np.array_equal(rx.view(torch.uint8).cpu().numpy(), ex)
    assert np.array_equal(rsf.cpu().numpy().view(np.uint32), es)
    # determinism: a second dispatch is bit-identical
    (rx2, rsf2), _, rw2, h2, _ = buf.dispatch(xg, topk_idx=tg, topk_weights=wg, **kw)
    assert torch.equal(rx2.view(torch.uint8), rx.view(torch.uint8)) and torch.equal(rsf2, rsf) and torch.equal(rw2, rw)
    assert torch.equal(h2.recv_src_metadata, handle.recv_src_metadata)
    # combine
    y = torch.randn((rx.size(0), H), generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    cx, cw, _ = buf.combine(y.to(DEV), handle, topk_weights=rw)
    torch.cuda.synchronize()
    ox, _ = O.combine_fast(y, torch.from_numpy(ew), lay['recv_src_metadata'], T, K)
    assert np.array_equal(bf16_bits(cx), bf16_bits(ox))
    assert torch.equal(cw.cpu(), w)
    # linearity: combine(2y) == 2 combine(y) exactly (powers of two commute with rounding)
    cx2, _, _ = buf.combine((y * 2).to(DEV), handle)
    assert torch.equal(cx2, cx * 2)
    buf.destroy()


def test_c5_one_gpu_share_of_ep32():
    T, H, E, K, A, R, rank = 16384, 7168, 256, 6, 128, 32, 5
    epr = E // R
    x = make_tokens(T, H, seed=0, outliers=True)
    topk, w = make_routing(T, E, K, seed=0)
    lay = O.rank_share_layout(topk.numpy(), E, R, rank, A, T)
    q, s = O.quantise(x)
    buf = _buffer(T, H, K, R=R, rank=rank, fp8=True)
    xg, tg, wg = x.to(DEV), topk.to(DEV), w.to(DEV)
    (rx, rsf), _, rw, handle, _ = buf.dispatch(xg, topk_idx=tg, topk_weights=wg, num_experts=E, expert_alignment=A,
                                               do_expand=True, do_zero_padding=True, fused_fp8_quant=True)
    torch.cuda.synchronize()
    for name in ('psum_num_recv_tokens_per_rank', 'psum_num_recv_tokens_per_expert',
                 'num_unaligned_recv_tokens_per_expert', 'dst_buffer_slot_idx', 'recv_src_metadata'):
        assert np.array_equal(getattr(handle, name).cpu().numpy(), lay[name]), name
    # the 32 partition-major regions: region r, slot s holds [fp8 row | scales | topk_idx | weights | src]
    tok = O.dispatch_token_layout(H, 2 * (H // 128), K)
    tb = tok.num_bytes()
    assert tb == 7488
    regions = buf.runtime.buffer_tensor()[:R * T * tb].view(R, T, tb)
    dst = handle.dst_buffer_slot_idx.long()
    part = torch.where(tg >= 0, tg // epr, torch.full_like(tg, -1))
    tt, jj = torch.nonzero(dst >= 0, as_tuple=True)
    rows = regions[part[tt, jj], dst[tt, jj]]
    assert rows.size(0) == int(lay['num_send_tokens_per_rank'].sum())
    qd, sd = q.to(DEV), s.to(DEV)
    assert torch.equal(rows[:, :H], qd[tt])
    assert torch.equal(rows[:, tok.sf_offset:tok.sf_offset + 224].contiguous().view(torch.float32), sd[tt])
    assert torch.equal(rows[:, tok.topk_idx_offset:tok.topk_idx_offset + 8 * K].contiguous().view(torch.int64), tg[tt])
    assert torch.equal(rows[:, tok.topk_weights_offset:tok.topk_weights_offset + 4 * K].contiguous().view(torch.float32), wg[tt])
    assert torch.equal(rows[:, tok.src_token_global_idx_offset:tok.src_token_global_idx_offset + 4].contiguous().view(torch.int32).flatten(),
                       (rank * T + tt).int())
    # expansion of the own region against the oracle
    ex, es, ew = O.rank_share_dispatch(q.numpy(), s.numpy().view(np.uint32), w.numpy(), lay)
    assert np.array_equal(rx.view(torch.uint8).cpu().numpy(), ex)
    assert np.array_equal(rsf.cpu().numpy().view(np.uint32), es)
    assert np.array_equal(rw.cpu().numpy().view(np.uint32), ew.view(np.uint32))

    # combine from a partition-major buffer: random partials at the master positions, deferred epilogue
    g = torch.Generator(device=DEV).manual_seed(7)
    ctb = O.combine_token_layout(H, K).num_bytes()
    G = min(K, R)
    arena = buf.runtime.buffer_tensor()
    cbuf = arena[:G * T * ctb].view(G * T, ctb)
    cbuf[:, :H * 2] = torch.randn((G * T, H), generator=g, device=DEV).to(torch.bfloat16).view(torch.uint8)
    wv = torch.zeros((G, T, K), dtype=torch.float32, device=DEV)
    for j in range(K):                      # group = top-k position (R >= K): its vector carries the positions
        same = (part == part[:, j:j + 1]) & (tg >= 0)        # that live on the same partition
        wv[j] = torch.where(same, wg, torch.zeros_like(wg))
    cbuf[:, H * 2:H * 2 + 4 * K] = wv.view(G * T, K).view(torch.uint8)
    y = torch.randn((rx.size(0), H), generator=g, device=DEV).to(torch.bfloat16)
    ev = buf.combine(y, handle, topk_weights=rw, async_with_compute_stream=True, defer_epilogue=True)
    cx, cw = ev.current_stream_wait()
    torch.cuda.synchronize()
    # reference on the GPU with torch fp32 ops in the same order: masters ascending, one rounding
    P = cbuf[:, :H * 2].contiguous().view(torch.bfloat16).view(G, T, H)
    later_same = torch.zeros_like(tg, dtype=torch.bool)
    for j in range(K):
        for j2 in range(j + 1, K):
            later_same[:, j] |= (part[:, j2] == part[:, j]) & (tg[:, j2] >= 0)
    master = (tg >= 0) & ~later_same
    nm = master.sum(dim=1)
    acc = torch.zeros((T, H), dtype=torch.float32, device=DEV)
    started = torch.zeros(T, dtype=torch.bool, device=DEV)
    for j in range(K):
        m = master[:, j]
        acc[m & ~started] = P[j][m & ~started].float()
        acc[m & started] = acc[m & started] + P[j][m & started].float()
        started |= m
    ref = acc.to(torch.bfloat16)
    one = nm == 1
    jone = master.float().argmax(dim=1)
    ref[one] = P[jone[one], torch.nonzero(one).flatten()]
    assert torch.equal(cx.view(torch.int16), ref.view(torch.int16))
    assert torch.equal(cw, wg)
    # the owner-side partials of this partition match the oracle on a sample of rows
    own_p, _ = O.combine_partial(y.cpu(), rw.cpu(), lay['recv_src_metadata'][:64], R, rank, T)
    for (grp, src), p in own_p.items():
        assert torch.equal(P[grp, src - rank * T].cpu().view(torch.int16), p.view(torch.int16))
    buf.destroy()


def test_ep32_node_full_size_properties():
    """The EP32 configuration with all 32 partitions on the GPU, each dispatching the full 16384 x 7168
    tokens (fused FP8) with a routing of its own: every partition receives its real share from 32 sources.
    Checked through properties that hold at any size: per-source counts, the received rows are the
    quantised source tokens bit for bit, slots tile the experts' aligned blocks, padding is zero, and the
    combine returns (number of selections) x (a small-integer row), exactly."""
    import deep_ep
    R, T, H, E, K, A = 32, 16384, 7168, 256, 6, 128
    El = E // R
    torch.cuda.empty_cache()
    free_bytes, _ = torch.cuda.mem_get_info()
    if free_bytes < 220 * (1 << 30):
        pytest.skip(f'needs about 200 GiB of free device memory (32 arenas of 3.9 GB and the tensors), {free_bytes >> 30} GiB free')
    node = deep_ep.LocalNode(R)
    bufs = []
    try:
        for r in range(R):
            bufs.append(deep_ep.EPBuffer(node.group(r), num_max_tokens_per_rank=T, hidden=H, num_topk=K,
                                         use_fp8_dispatch=True, explicitly_destroy=True))
        _ep32_node_checks(bufs, R, T, H, E, K, A, El)
    finally:
        torch.cuda.synchronize()
        for b in bufs:
            b.destroy()


def _ep32_node_checks(bufs, R, T, H, E, K, A, El):
    x = make_tokens(T, H, seed=0, outliers=True)
    q, s = O.quantise(x)                                         # CPU quantiser = the reference's arithmetic
    qg, sg, xg = q.to(DEV), s.to(DEV), x.to(DEV)
    base_topk, base_w = make_routing(T, E, K, seed=0, masked=0.05)
    # partition r routes token t like the base routing of token (t + 97 r) mod T, experts rotated by r
    topks, wts = [], []
    for r in range(R):
        t_ = torch.roll(base_topk, shifts=-97 * r, dims=0)
        topks.append(torch.where(t_ >= 0, (t_ + r) % E, t_).to(DEV))
        wts.append(torch.roll(base_w, shifts=-97 * r, dims=0).to(DEV))

    events = [bufs[r].dispatch(xg, topk_idx=topks[r], topk_weights=wts[r], num_experts=E, num_max_tokens_per_rank=T,
                               expert_alignment=A, do_expand=True, do_zero_padding=True, fused_fp8_quant=True,
                               async_with_compute_stream=True, defer_epilogue=True) for r in range(R)]
    z = (torch.arange(T, device=DEV).view(T, 1) * 3 + torch.arange(H, device=DEV).view(1, H)) % 7 - 3
    z = z.to(torch.bfloat16)                                      # "expert output" of a token: small integers
    handles, partial_events = [], []
    all_topk = torch.stack(topks)                                 # [R, T, K]
    for d in range(R):
        (rx, rsf), _, rw, handle = events[d].current_stream_wait()
        meta = handle.recv_src_metadata.long()
        slots, src = meta[:, :K], meta[:, K]
        src_rank, src_tok = src // T, src % T
        # per source: exactly its tokens with a selection on partition d, in token order
        psum = [0] + handle.psum_num_recv_tokens_per_rank.tolist()
        local_any = ((all_topk >= d * El) & (all_topk < (d + 1) * El)).any(dim=2)     # [R, T]
        assert psum[1:] == torch.cumsum(local_any.sum(dim=1), 0).tolist()
        for sr in (0, d, R - 1):
            part = slice(psum[sr], psum[sr + 1])
            assert torch.equal(src_tok[part], local_any[sr].nonzero().flatten())
            assert bool((src_rank[part] == sr).all())
        sel = all_topk[src_rank, src_tok]                           # [N, K] global expert ids
        local = (sel >= d * El) & (sel < (d + 1) * El)
        assert torch.equal(slots >= 0, local)
        flat = slots[local]
        assert torch.unique(flat).numel() == flat.numel() == int(handle.num_unaligned_recv_tokens_per_expert.sum())
        tok_of_slot = src_tok.unsqueeze(1).expand(-1, K)[local]
        assert torch.equal(rx.view(torch.uint8)[flat], qg[tok_of_slot])
        assert torch.equal(rsf[flat], sg[tok_of_slot])
        assert torch.equal(rw[flat], torch.stack(wts)[src_rank, src_tok][local])
        pad = torch.ones(rx.size(0), dtype=torch.bool, device=DEV)
        pad[flat] = False
        assert int(rx.view(torch.uint8)[pad].count_nonzero()) == 0 and int(rsf[pad].count_nonzero()) == 0
        cnt = handle.num_unaligned_recv_tokens_per_expert.long()
        start = handle.psum_num_recv_tokens_per_expert.long() - cnt
        assert bool((start % A == 0).all())
        assert torch.equal(cnt, torch.bincount(sel[local] - d * El, minlength=El))
        # experts are the identity on z: row of (source token, j) = z[token]
        y = torch.full((rx.size(0), H), 99.0, dtype=torch.bfloat16, device=DEV)
        y[flat] = z[tok_of_slot]
        handles.append((handle, y, rw))
        del rx, rsf
    # every partition has expanded what it received: only now may the combine reuse the buffers
    for d, (handle, y, rw) in enumerate(handles):
        partial_events.append(bufs[d].combine(y, handle, topk_weights=rw, async_with_compute_stream=True,
                                              defer_epilogue=True))
    del handles
    for r in range(R):
        cx, cw = partial_events[r].current_stream_wait()
        n_sel = (topks[r] >= 0).sum(dim=1, keepdim=True).to(torch.float32)
        assert torch.equal(cx.float(), z.float() * n_sel), r      # small integers: every sum and rounding is exact
        assert torch.equal(cw, wts[r])


def test_65536_tokens_reach_the_scanned_layout_by_size():
    """Four times the headline's tokens: 512 layout workgroups (beyond what the slot assignment folds itself, so the
    scan kernel runs without any tuning knob being touched), 3.7 million wave tasks in the copy kernel.  Layout
    against the oracle; payload, scales and padding through the layout's own properties; combine through a round
    trip: the rows of a token are copies of it, so their sum is top-k times the token (exact in BF16 at top-4)."""
    T, H, E, K, A = 65536, 2048, 256, 4, 128
    x = make_tokens(T, H, seed=4, outliers=True)
    topk, w = make_routing(T, E, K, seed=4)
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    buf = _buffer(T, H, K)                        # sized for BF16 rows: the FP8 dispatch fits as well
    xg, tg, wg = x.to(DEV), topk.to(DEV), w.to(DEV)
    (rx, rsf), _, rw, handle, _ = buf.dispatch(xg, topk_idx=tg, topk_weights=wg, num_experts=E, expert_alignment=A,
                                               do_expand=True, do_zero_padding=True, fused_fp8_quant=True)
    torch.cuda.synchronize()
    assert handle.num_expanded_tokens == lay['num_expanded_tokens'] == rx.size(0)
    assert np.array_equal(handle.recv_src_metadata.cpu().numpy(), lay['recv_src_metadata'])
    assert np.array_equal(handle.psum_num_recv_tokens_per_expert.cpu().numpy(), lay['psum_num_recv_tokens_per_expert'])
    assert np.array_equal(handle.dst_buffer_slot_idx.cpu().numpy(), lay['dst_buffer_slot_idx'])
    q, s = O.quantise(x)
    _check_layout_properties(handle, tg, E, A, rx.view(torch.uint8), q.to(DEV))
    _check_layout_properties(handle, tg, E, A, rsf.view(torch.int32), s.view(torch.int32).to(DEV))
    # BF16 round trip: dispatch the rows verbatim, combine the copies
    rb, _, rwb, hb, _ = buf.dispatch(xg, topk_idx=tg, topk_weights=wg, num_experts=E, expert_alignment=A,
                                     do_expand=True, do_zero_padding=True)
    assert torch.equal(hb.recv_src_metadata, handle.recv_src_metadata)
    cx, cw, _ = buf.combine(rb, hb, topk_weights=rwb)
    torch.cuda.synchronize()
    assert torch.equal(cx, xg * K)
    assert torch.equal(cw, wg)
    buf.destroy()
