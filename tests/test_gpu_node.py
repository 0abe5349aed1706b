"""Every partition of an EP group on this one GPU, connected into a node: the dispatch of partition s
puts its packed rows and row counts straight into the arena of the partition they are for, the
receive side of each partition lays out whatever arrived, and the combine sends every partial back
to the arena its token came from.  Driven phase by phase through the deferred epilogues of the
reference API, on one stream.  Checked against the multi-rank oracle and against the vectors the
reference's own refs.dispatch / refs.combine produced under 2- and 4-rank gloo groups.
"""
import os

import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_routing, make_tokens
from oracle import ep_oracle as O

pytestmark = pytest.mark.gpu
DEV = 'cuda'
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')


def make_node(R, max_tokens, H, K, fp8):
    import deep_ep
    node = deep_ep.LocalNode(R)
    return [deep_ep.EPBuffer(node.group(r), num_max_tokens_per_rank=max_tokens, hidden=H, num_topk=K,
                             use_fp8_dispatch=fp8, explicitly_destroy=True) for r in range(R)]


def dispatch_all(bufs, xs, topks, ws, **kw):
    events = [b.dispatch(x, topk_idx=t, topk_weights=w, async_with_compute_stream=True, defer_epilogue=True, **kw)
              for b, x, t, w in zip(bufs, xs, topks, ws)]                  # send side of every partition
    return [ev.current_stream_wait() for ev in events]                    # then every receive side


def combine_all(bufs, ys, handles, weights, biases):
    events = [b.combine(y, h, topk_weights=w, bias=bias, async_with_compute_stream=True, defer_epilogue=True)
              for b, y, h, w, bias in zip(bufs, ys, handles, weights, biases)]   # owner-side partials everywhere
    return [ev.current_stream_wait() for ev in events]                           # then the token-side reduces


def oracle_dispatch(rows, sfs, topks, ws, E, R, A, max_tokens):
    """Per destination: the received stream parsed back into its parts, and its layout."""
    K = topks[0].shape[1]
    HB = rows[0].shape[1]
    SB = 0 if sfs[0] is None else sfs[0].shape[1]
    tok = O.dispatch_token_layout(HB, SB // 2, K)
    sends = [O.send_layout(t, E, R) for t in topks]
    regions = [O.pack_regions(rows[s], sfs[s], topks[s], ws[s], sends[s][0], sends[s][1], E, R, s, max_tokens)
               for s in range(R)]
    out = []
    for d in range(R):
        stream = np.concatenate([regions[s][d] for s in range(R)], axis=0)
        counts = [regions[s][d].shape[0] for s in range(R)]
        idx = stream[:, tok.topk_idx_offset:tok.topk_idx_offset + 8 * K].copy().view(np.int64)
        w = stream[:, tok.topk_weights_offset:tok.topk_weights_offset + 4 * K].copy().view(np.float32)
        src = stream[:, tok.src_token_global_idx_offset:tok.src_token_global_idx_offset + 4].copy().view(np.int32)[:, 0]
        lay = O.recv_layout(idx, src, counts, E, R, d, A)
        hid = stream[:, :HB]
        sf = stream[:, tok.sf_offset:tok.sf_offset + SB] if SB else None
        ex, es, ew = O.expand(hid, sf, w, lay['recv_src_metadata'], lay['num_expanded_tokens'])
        out.append(dict(lay=lay, x=ex, sf=es, w=ew, stream=stream, counts=counts))
    return sends, out


NODE_CASES = [
    # R, max_tokens, H, E, K, A, masked
    (2, 96, 256, 8, 3, 1, 0.0),
    (4, 150, 512, 32, 6, 16, 0.15),        # R < K: partial groups are partitions
    (8, 70, 256, 64, 4, 128, 0.2),         # R >= K: partial groups are top-k positions
    (3, 260, 384, 12, 5, 8, 0.3),          # receive streams longer than one layout block
]


# the host sync does not interact with the input format: pre-quantised input runs with it only
NODE_MODES = [(m, s) for m in ('bf16', 'fp8_fused', 'fp8_prequant', 'fp8_fused_colmajor') for s in (True, False)
              if s or m != 'fp8_prequant']


@pytest.mark.parametrize('R,max_tokens,H,E,K,A,masked', NODE_CASES)
@pytest.mark.parametrize('mode,do_cpu_sync', NODE_MODES)
def test_node_dispatch_combine(R, max_tokens, H, E, K, A, masked, mode, do_cpu_sync):
    col_major = mode.endswith('_colmajor')          # scales asked for as columns; compared as values
    mode = mode.replace('_colmajor', '')
    bufs = make_node(R, max_tokens, H, K, mode != 'bf16')
    Ts = [max(1, max_tokens - 7 * r) for r in range(R)]                   # ragged token counts
    xs = [make_tokens(T, H, seed=10 * R + r, outliers=True) for r, T in enumerate(Ts)]
    routing = [make_routing(T, E, K, seed=20 * R + r, masked=masked) for r, T in enumerate(Ts)]
    topks, ws = [t for t, _ in routing], [w for _, w in routing]
    quant = [O.quantise(x) for x in xs]
    if mode == 'bf16':
        rows = [bf16_bits(x).view(np.uint8).reshape(x.size(0), -1) for x in xs]
        sfs = [None] * R
        gx = [x.to(DEV) for x in xs]
    else:
        rows = [q.numpy() for q, _ in quant]
        sfs = [s.numpy().view(np.uint8).reshape(s.size(0), -1) for _, s in quant]
        gx = [x.to(DEV) for x in xs] if mode == 'fp8_fused' else \
            [(q.view(torch.float8_e4m3fn).to(DEV), s.view(torch.int16).to(DEV)) for q, s in quant]
    sends, want = oracle_dispatch(rows, sfs, [t.numpy() for t in topks], [w.numpy() for w in ws], E, R, A, max_tokens)

    stats = [torch.zeros(E // R, dtype=torch.int32, device=DEV) for _ in range(R)]
    events = [bufs[r].dispatch(gx[r], topk_idx=topks[r].to(DEV), topk_weights=ws[r].to(DEV),
                               cumulative_local_expert_recv_stats=stats[r], num_experts=E,
                               num_max_tokens_per_rank=max_tokens, expert_alignment=A, do_expand=True,
                               do_zero_padding=True, do_cpu_sync=do_cpu_sync, async_with_compute_stream=True,
                               defer_epilogue=True, fused_fp8_quant=mode == 'fp8_fused',
                               use_tma_aligned_col_major_sf=col_major) for r in range(R)]
    outs = [ev.current_stream_wait() for ev in events]
    torch.cuda.synchronize()

    handles = []
    for r, (recv, _, rw, handle) in enumerate(outs):
        lay = want[r]['lay']
        n, ne = lay['num_recv_tokens'], lay['num_expanded_tokens']
        assert np.array_equal(handle.dst_buffer_slot_idx.cpu().numpy(), sends[r][0])
        assert np.array_equal(handle.psum_num_recv_tokens_per_rank.cpu().numpy(), lay['psum_num_recv_tokens_per_rank'])
        assert np.array_equal(handle.psum_num_recv_tokens_per_expert.cpu().numpy(), lay['psum_num_recv_tokens_per_expert'])
        assert np.array_equal(handle.num_unaligned_recv_tokens_per_expert.cpu().numpy(),
                              lay['num_unaligned_recv_tokens_per_expert'])
        assert np.array_equal(stats[r].cpu().numpy(), lay['num_unaligned_recv_tokens_per_expert'])
        assert np.array_equal(handle.recv_src_metadata.cpu().numpy()[:n], lay['recv_src_metadata'])
        if do_cpu_sync:
            assert handle.num_recv_tokens == n and handle.num_expanded_tokens == ne
            assert handle.num_recv_tokens_per_expert_list == lay['num_recv_tokens_per_expert_list']
            assert handle.recv_src_metadata.size(0) == n
        else:
            assert (handle.num_recv_tokens, handle.num_expanded_tokens) == O.no_sync_sizes(R, max_tokens, K, E, A)
        rx, rsf = recv if isinstance(recv, tuple) else (recv, None)
        assert np.array_equal(rx.view(torch.uint8).cpu().numpy().reshape(rx.size(0), -1)[:ne], want[r]['x'])
        if rsf is not None:
            assert rsf.stride() == ((1, rsf.size(0)) if col_major else (rsf.size(1), 1))
            # (numpy makes the copy row-major: torch calls a single column of any stride contiguous already)
            assert np.array_equal(np.ascontiguousarray(rsf.cpu().numpy()).view(np.uint8).reshape(rsf.size(0), -1)[:ne],
                                  want[r]['sf'])
        assert np.array_equal(rw.cpu().numpy().view(np.uint32)[:ne], want[r]['w'].view(np.uint32))
        handles.append(handle)

    # cached replay through the node: new payload and weights, the layout of the handles (packed rows then
    # carry no routing metadata, which moves the scales and the weights inside them)
    xs2 = [make_tokens(T, H, seed=30 * R + r) for r, T in enumerate(Ts)]
    ws2 = [torch.randn(w.shape, generator=torch.Generator().manual_seed(r)).masked_fill(topks[r] < 0, 0)
           for r, w in enumerate(ws)]
    quant2 = [O.quantise(x) for x in xs2]
    if mode == 'bf16':
        rows2 = [bf16_bits(x).view(np.uint8).reshape(x.size(0), -1) for x in xs2]
        sfs2 = [None] * R
        gx2 = [x.to(DEV) for x in xs2]
    else:
        rows2 = [q.numpy() for q, _ in quant2]
        sfs2 = [s_.numpy().view(np.uint8).reshape(s_.size(0), -1) for _, s_ in quant2]
        gx2 = [x.to(DEV) for x in xs2] if mode == 'fp8_fused' else \
            [(q.view(torch.float8_e4m3fn).to(DEV), s_.view(torch.int16).to(DEV)) for q, s_ in quant2]
    _, want2 = oracle_dispatch(rows2, sfs2, [t.numpy() for t in topks], [w.numpy() for w in ws2], E, R, A, max_tokens)
    evs = [bufs[r].dispatch(gx2[r], topk_weights=ws2[r].to(DEV), handle=handles[r], do_expand=True,
                            do_zero_padding=True, async_with_compute_stream=True, defer_epilogue=True,
                            fused_fp8_quant=mode == 'fp8_fused', use_tma_aligned_col_major_sf=col_major)
           for r in range(R)]
    outs2 = [ev.current_stream_wait() for ev in evs]
    torch.cuda.synchronize()
    for r, (recv2, _, rw2, h2) in enumerate(outs2):
        assert h2 is handles[r]
        ne = want[r]['lay']['num_expanded_tokens']
        rx2, rsf2 = recv2 if isinstance(recv2, tuple) else (recv2, None)
        assert np.array_equal(rx2.view(torch.uint8).cpu().numpy().reshape(rx2.size(0), -1)[:ne], want2[r]['x'])
        if rsf2 is not None:
            assert np.array_equal(np.ascontiguousarray(rsf2.cpu().numpy()).view(np.uint8).reshape(rsf2.size(0), -1)[:ne],
                                  want2[r]['sf'])
        assert np.array_equal(rw2.cpu().numpy().view(np.uint32)[:ne], want2[r]['w'].view(np.uint32))

    # combine: every owner reduces what it received and sends the partial home
    g = torch.Generator().manual_seed(R)
    ys = [torch.randn((outs[r][0][0].size(0) if isinstance(outs[r][0], tuple) else outs[r][0].size(0), H),
                      generator=g).to(torch.bfloat16) for r in range(R)]
    for nbias in (0, 2):
        biases = [[torch.randn((Ts[r], H), generator=g).to(torch.bfloat16) for _ in range(nbias)] for r in range(R)]
        cevs = [bufs[r].combine(ys[r].to(DEV), handles[r], topk_weights=outs[r][2],
                                bias=tuple(b.to(DEV) for b in biases[r]) if nbias else None,
                                async_with_compute_stream=True, defer_epilogue=True) for r in range(R)]
        res = [ev.current_stream_wait() for ev in cevs]
        torch.cuda.synchronize()
        parts, wvecs = {}, {}
        for r in range(R):
            lay = want[r]['lay']
            p, wv = O.combine_partial(ys[r], torch.from_numpy(want[r]['w']), lay['recv_src_metadata'], R, r, max_tokens)
            assert not set(p) & set(parts)
            parts.update(p)
            wvecs.update(wv)
        for s in range(R):
            ox, ow = O.combine_final(topks[s].numpy(), E, R, s, max_tokens, lambda k: parts[k], lambda k: wvecs[k],
                                     biases[s][0] if nbias else None, biases[s][1] if nbias else None, H, True)
            cx, cw = res[s]
            assert np.array_equal(bf16_bits(cx), bf16_bits(ox)), (nbias, s)
            assert torch.equal(cw.cpu(), ow) and torch.equal(cw.cpu(), ws[s])
    for b in bufs:
        b.destroy()


def test_node_reproduces_the_reference_dispatch_vectors():
    """tests/golden/dispatch_golden_w2.npz: inputs of both ranks and what refs.dispatch gave each of them
    (received rows in source order, local expert ids, weights, source tokens, per-source counts)."""
    g = np.load(os.path.join(GOLD, 'dispatch_golden_w2.npz'))
    R = 2
    T0, K, E, H, max_tokens, world = g['r0.cfg'].tolist()
    assert world == R
    bufs = make_node(R, max_tokens, H, K, False)
    xs = [torch.from_numpy(g[f'r{r}.x'].view(np.int16)).view(torch.bfloat16) for r in range(R)]
    topks = [torch.from_numpy(g[f'r{r}.topk_idx']) for r in range(R)]
    ws = [torch.from_numpy(g[f'r{r}.topk_weights']) for r in range(R)]
    outs = dispatch_all(bufs, [x.to(DEV) for x in xs], [t.to(DEV) for t in topks], [w.to(DEV) for w in ws],
                        num_experts=E, num_max_tokens_per_rank=max_tokens, expert_alignment=4, do_expand=True,
                        do_zero_padding=True)
    torch.cuda.synchronize()
    epr = E // R
    for d, (rx, _, rw, handle) in enumerate(outs):
        counts = g[f'r{d}.num_recv_tokens_per_rank']
        assert np.array_equal(handle.psum_num_recv_tokens_per_rank.cpu().numpy(), np.cumsum(counts))
        meta = handle.recv_src_metadata.cpu().numpy()
        assert np.array_equal(meta[:, K], g[f'r{d}.recv_src_token_idx'])
        want_idx = g[f'r{d}.recv_topk_idx']                      # local expert id or -1
        assert np.array_equal(meta[:, :K] >= 0, want_idx >= 0)
        psum = np.concatenate([[0], handle.psum_num_recv_tokens_per_expert.cpu().numpy()])
        got_x, got_w = bf16_bits(rx), rw.cpu().numpy()
        for i in range(meta.shape[0]):
            for j in range(K):
                s = meta[i, j]
                if s < 0:
                    continue
                e = want_idx[i, j]
                assert (psum[e] + 3) // 4 * 4 <= s < psum[e + 1]        # inside the expert's aligned block
                assert np.array_equal(got_x[s], g[f'r{d}.recv_x'][i])
                assert got_w[s] == g[f'r{d}.recv_topk_weights'][i, j]
        for e in range(epr):
            assert psum[e + 1] - (psum[e] + 3) // 4 * 4 == int((want_idx == e).sum())
    for b in bufs:
        b.destroy()


@pytest.mark.parametrize('world', [2, 4])
def test_node_reproduces_the_reference_combine_vectors(world):
    """tests/golden/combine_golden_w{2,4}.npz: expert outputs per (token, selection) of rank 0's tokens and
    what refs.combine(reduce_in_local=True) made of them."""
    g = np.load(os.path.join(GOLD, f'combine_golden_w{world}.npz'))
    for ci in range(5):
        p = f'w{world}.c{ci}.'
        T, K, E, H, nbias, W = g[p + 'cfg'].tolist()
        assert W == world
        bufs = make_node(W, T, H, K, False)
        topk = torch.from_numpy(g[p + 'topk_idx'])
        y3 = torch.from_numpy(g[p + 'y'].view(np.int16)).view(torch.bfloat16)          # [T, K, H]
        bias = [torch.from_numpy(g[p + f'bias{b}'].view(np.int16)).view(torch.bfloat16) for b in range(nbias)]
        # rank 0 owns the tokens; the other ranks dispatch a single token that selects nothing
        xs = [torch.zeros((T if r == 0 else 1, H), dtype=torch.bfloat16) for r in range(W)]
        topks = [topk if r == 0 else torch.full((1, K), -1, dtype=torch.int64) for r in range(W)]
        ws = [torch.zeros(t.shape, dtype=torch.float32) for t in topks]
        outs = dispatch_all(bufs, [x.to(DEV) for x in xs], [t.to(DEV) for t in topks], [w.to(DEV) for w in ws],
                            num_experts=E, num_max_tokens_per_rank=T, expert_alignment=2, do_expand=True,
                            do_zero_padding=True)
        torch.cuda.synchronize()
        ys = []
        for r, (rx, _, _, handle) in enumerate(outs):
            meta = handle.recv_src_metadata.cpu().numpy()
            y = torch.full((rx.size(0), H), 7.0, dtype=torch.bfloat16)              # padding rows hold garbage
            for i in range(meta.shape[0]):
                for j in range(K):
                    if meta[i, j] >= 0:
                        y[meta[i, j]] = y3[meta[i, K], j]
            ys.append(y.to(DEV))
        handles = [o[3] for o in outs]
        biases = [(tuple(b.to(DEV) for b in bias) if nbias == 2 else bias[0].to(DEV)) if (r == 0 and nbias) else
                  (None if nbias == 0 else (tuple(torch.zeros((1, H), dtype=torch.bfloat16, device=DEV) for _ in range(2))
                                            if nbias == 2 else torch.zeros((1, H), dtype=torch.bfloat16, device=DEV)))
                  for r in range(W)]
        res = combine_all(bufs, ys, handles, [None] * W, biases)
        torch.cuda.synchronize()
        got, want = bf16_bits(res[0][0]), g[p + 'out']
        # the reference zeroes masked selections and adds exact zeros: only the sign of a zero may differ
        same = (got == want) | (((got | want) & 0x7fff) == 0)
        assert same.all(), (world, ci)
        for b in bufs:
            b.destroy()


def test_node_with_an_empty_partition_and_disconnect():
    """A partition without tokens still takes part (it receives and reduces for the others); destroying a
    partition leaves the rest usable on their own."""
    R, max_tokens, H, E, K, A = 2, 40, 128, 4, 2, 4
    bufs = make_node(R, max_tokens, H, K, False)
    Ts = [33, 0]
    xs = [make_tokens(T, H, seed=r) if T else torch.empty((0, H), dtype=torch.bfloat16) for r, T in enumerate(Ts)]
    routing = [make_routing(T, E, K, seed=r) if T else (torch.empty((0, K), dtype=torch.int64),
                                                         torch.empty((0, K), dtype=torch.float32))
               for r, T in enumerate(Ts)]
    topks, ws = [t for t, _ in routing], [w for _, w in routing]
    rows = [bf16_bits(x).view(np.uint8).reshape(x.size(0), H * 2) for x in xs]
    _, want = oracle_dispatch(rows, [None] * R, [t.numpy() for t in topks], [w.numpy() for w in ws], E, R, A, max_tokens)
    outs = dispatch_all(bufs, [x.to(DEV) for x in xs], [t.to(DEV) for t in topks], [w.to(DEV) for w in ws],
                        num_experts=E, num_max_tokens_per_rank=max_tokens, expert_alignment=A, do_expand=True,
                        do_zero_padding=True)
    torch.cuda.synchronize()
    for r, (rx, _, rw, handle) in enumerate(outs):
        assert np.array_equal(handle.recv_src_metadata.cpu().numpy(), want[r]['lay']['recv_src_metadata'])
        assert np.array_equal(rx.view(torch.uint8).cpu().numpy().reshape(rx.size(0), H * 2), want[r]['x'])
    ys = [o[0] for o in outs]                                   # identity experts
    res = combine_all(bufs, ys, [o[3] for o in outs], [o[2] for o in outs], [None] * R)
    torch.cuda.synchronize()
    # every token selected K distinct experts: the sum of K copies
    expect = (xs[0].float() * K).to(torch.bfloat16)
    assert torch.equal(res[0][0].cpu().view(torch.int16), expect.view(torch.int16))
    assert torch.equal(res[0][1].cpu(), ws[0]) and res[1][0].size(0) == 0

    bufs[1].destroy()
    x = xs[0].to(DEV)
    rx, _, rw, handle, _ = bufs[0].dispatch(x, topk_idx=topks[0].to(DEV), topk_weights=ws[0].to(DEV), num_experts=E,
                                            num_max_tokens_per_rank=max_tokens, expert_alignment=A, do_expand=True,
                                            do_zero_padding=True)
    torch.cuda.synchronize()
    lay = O.rank_share_layout(topks[0].numpy(), E, R, 0, A, max_tokens)
    assert np.array_equal(handle.recv_src_metadata.cpu().numpy(), lay['recv_src_metadata'])
    bufs[0].destroy()


def test_node_hand_derived_two_rank_example():
    """A case small enough to derive by hand from the reference's code: R=2, E=4, K=2, A=2, maxT=4; rank 0
    holds three tokens with topk_idx [[0,1],[3,-1],[2,0]], rank 1 holds none.  Expected values are written
    out literally, not computed by the oracle."""
    R, max_tokens, H, E, K, A = 2, 4, 64, 4, 2, 2
    bufs = make_node(R, max_tokens, H, K, False)
    x0 = make_tokens(3, H, seed=5)
    topk0 = torch.tensor([[0, 1], [3, -1], [2, 0]], dtype=torch.int64)
    w0 = torch.tensor([[0.25, 0.75], [1.0, 0.0], [0.5, 0.5]], dtype=torch.float32)
    xs = [x0, torch.empty((0, H), dtype=torch.bfloat16)]
    topks = [topk0, torch.empty((0, K), dtype=torch.int64)]
    ws = [w0, torch.empty((0, K), dtype=torch.float32)]
    outs = dispatch_all(bufs, [x.to(DEV) for x in xs], [t.to(DEV) for t in topks], [w.to(DEV) for w in ws],
                        num_experts=E, num_max_tokens_per_rank=max_tokens, expert_alignment=A, do_expand=True,
                        do_zero_padding=True)
    torch.cuda.synchronize()
    (rx0, _, rw0, h0), (rx1, _, rw1, h1) = outs
    zero = torch.zeros(H, dtype=torch.bfloat16)
    # rank 0: receives t0 (experts 0 and 1) and t2 (expert 0 at j=1)
    assert h0.dst_buffer_slot_idx.tolist() == [[-1, 0], [0, -1], [1, 1]]
    assert h0.psum_num_recv_tokens_per_rank.tolist() == [2, 2]
    assert h0.num_unaligned_recv_tokens_per_expert.tolist() == [2, 1]
    assert h0.psum_num_recv_tokens_per_expert.tolist() == [2, 3]
    assert (h0.num_recv_tokens, h0.num_expanded_tokens, h0.num_recv_tokens_per_expert_list) == (2, 4, [2, 2])
    assert h0.recv_src_metadata.tolist() == [[0, 2, 0, 1], [-1, 1, 2, 1]]
    assert torch.equal(rx0.cpu(), torch.stack([x0[0], x0[2], x0[0], zero]))
    assert rw0.tolist() == [0.25, 0.5, 0.75, 0.0]
    # rank 1: receives t1 (expert 3 = local 1) and t2 (expert 2 = local 0)
    assert h1.psum_num_recv_tokens_per_rank.tolist() == [2, 2]
    assert h1.num_unaligned_recv_tokens_per_expert.tolist() == [1, 1]
    assert h1.psum_num_recv_tokens_per_expert.tolist() == [1, 3]
    assert h1.recv_src_metadata.tolist() == [[2, -1, 1, 0], [0, -1, 2, 0]]
    assert torch.equal(rx1.cpu(), torch.stack([x0[2], zero, x0[1], zero]))
    assert rw1.tolist() == [0.5, 0.0, 1.0, 0.0]

    g = torch.Generator().manual_seed(1)
    y0 = torch.randn((4, H), generator=g).to(torch.bfloat16)
    y1 = torch.randn((4, H), generator=g).to(torch.bfloat16)
    b0 = torch.randn((3, H), generator=g).to(torch.bfloat16)
    b1 = torch.randn((3, H), generator=g).to(torch.bfloat16)
    empty_bias = tuple(torch.empty((0, H), dtype=torch.bfloat16, device=DEV) for _ in range(2))
    res = combine_all(bufs, [y0.to(DEV), y1.to(DEV)], [h0, h1], [rw0, rw1], [(b0.to(DEV), b1.to(DEV)), empty_bias])
    torch.cuda.synchronize()
    cx, cw = res[0]
    p_t0 = (y0[0].float() + y0[2].float()).to(torch.bfloat16)           # owner 0, two local slots
    bias = b0.float() + b1.float()
    want = torch.stack([
        (bias[0] + p_t0.float()).to(torch.bfloat16),
        (bias[1] + y1[2].float()).to(torch.bfloat16),                       # t1: one master, partial = y1[2] verbatim
        (bias[2] + y1[0].float() + y0[1].float()).to(torch.bfloat16),       # t2: masters j=0 (rank 1) then j=1 (rank 0)
    ])
    assert torch.equal(cx.cpu().view(torch.int16), want.view(torch.int16))
    assert torch.equal(cw.cpu(), w0)
    for b in bufs:
        b.destroy()


def test_partitions_connected_by_address():
    """ep_buffer_set_peers: the connection a process per GPU would make with mapped arena addresses, here
    with the addresses of three buffers of this process; same results as a node."""
    import deep_ep
    R, max_tokens, H, E, K, A = 3, 50, 128, 6, 3, 4
    bufs = [deep_ep.EPBuffer(deep_ep.LocalGroup(r, R), num_max_tokens_per_rank=max_tokens, hidden=H, num_topk=K,
                             explicitly_destroy=True) for r in range(R)]
    bases = [b.runtime.region(0)[0] for b in bufs]
    for b in bufs:
        b.runtime.set_peers(bases)
    Ts = [50, 41, 17]
    xs = [make_tokens(T, H, seed=60 + r) for r, T in enumerate(Ts)]
    routing = [make_routing(T, E, K, seed=70 + r, masked=0.1) for r, T in enumerate(Ts)]
    topks, ws = [t for t, _ in routing], [w for _, w in routing]
    rows = [bf16_bits(x).view(np.uint8).reshape(x.size(0), H * 2) for x in xs]
    _, want = oracle_dispatch(rows, [None] * R, [t.numpy() for t in topks], [w.numpy() for w in ws], E, R, A, max_tokens)
    outs = dispatch_all(bufs, [x.to(DEV) for x in xs], [t.to(DEV) for t in topks], [w.to(DEV) for w in ws],
                        num_experts=E, num_max_tokens_per_rank=max_tokens, expert_alignment=A, do_expand=True,
                        do_zero_padding=True)
    torch.cuda.synchronize()
    for r, (rx, _, rw, handle) in enumerate(outs):
        assert np.array_equal(handle.recv_src_metadata.cpu().numpy(), want[r]['lay']['recv_src_metadata'])
        assert np.array_equal(rx.view(torch.uint8).cpu().numpy().reshape(rx.size(0), H * 2), want[r]['x'])
    res = combine_all(bufs, [o[0] for o in outs], [o[3] for o in outs], [o[2] for o in outs], [None] * R)
    torch.cuda.synchronize()
    for r in range(R):
        n_sel = (topks[r] >= 0).sum(dim=1, keepdim=True)
        # identity experts: every partial is a sum of copies of the token; compare with the oracle's two-level sum
        parts, wv = {}, {}
        for d in range(R):
            p, w_ = O.combine_partial(torch.from_numpy(want[d]['x'].view(np.int16)).view(torch.bfloat16),
                                      torch.from_numpy(want[d]['w']), want[d]['lay']['recv_src_metadata'], R, d, max_tokens)
            parts.update(p)
            wv.update(w_)
        ox, ow = O.combine_final(topks[r].numpy(), E, R, r, max_tokens, lambda k: parts[k], lambda k: wv[k],
                                 None, None, H, True)
        assert np.array_equal(bf16_bits(res[r][0]), bf16_bits(ox)) and n_sel.numel() == Ts[r]
        assert torch.equal(res[r][1].cpu(), ow)
    for b in bufs:
        b.runtime.set_peers(None)
        b.destroy()


def test_node_phase_order_is_checked_on_the_host():
    """Nothing on the device waits across partitions, so the library refuses a phase whose peers have not
    enqueued the phase before it: a blocking dispatch inside a node, a combine before every partition has
    expanded."""
    import deep_ep
    R, max_tokens, H, E, K = 2, 16, 64, 4, 2
    bufs = make_node(R, max_tokens, H, K, False)
    xs = [make_tokens(max_tokens, H, seed=r).to(DEV) for r in range(R)]
    routing = [make_routing(max_tokens, E, K, seed=r) for r in range(R)]
    kw = dict(num_experts=E, num_max_tokens_per_rank=max_tokens, do_expand=True, do_zero_padding=True)
    # partition 0 wants its receive side before partition 1 has sent anything
    with pytest.raises(deep_ep._C.EPException, match='partition 1 of the node'):
        bufs[0].dispatch(xs[0], topk_idx=routing[0][0].to(DEV), topk_weights=routing[0][1].to(DEV), **kw)
    ev1 = bufs[1].dispatch(xs[1], topk_idx=routing[1][0].to(DEV), topk_weights=routing[1][1].to(DEV),
                           async_with_compute_stream=True, defer_epilogue=True, **kw)
    # partition 0's send is enqueued (the failed call got that far); its receive side can run now
    with pytest.raises(deep_ep._C.EPException, match='previous dispatch'):
        bufs[0].dispatch(xs[0], topk_idx=routing[0][0].to(DEV), topk_weights=routing[0][1].to(DEV),
                         async_with_compute_stream=True, defer_epilogue=True, **kw)       # peers have not expanded yet
    rx1, _, rw1, h1 = ev1.current_stream_wait()
    # combine of partition 1 before partition 0 has expanded what it received
    with pytest.raises(deep_ep._C.EPException, match='copy epilogue before any combine'):
        bufs[1].combine(rx1, h1, topk_weights=rw1, async_with_compute_stream=True, defer_epilogue=True)
    torch.cuda.synchronize()
    for b in bufs:
        b.destroy()


def test_node_rejects_scaled_rows_that_would_overlap():
    """Packed rows place the scales at the next multiple of 32 bytes behind the payload while their size adds
    the payload unaligned (layout/ep/token.hpp:36-43,59-61): with 144 FP8 bytes a row, the metadata of row s
    would land in row s + 1.  The host refuses instead of corrupting the regions."""
    import deep_ep
    R, T, H, E, K = 2, 16, 144, 8, 4
    bufs = make_node(R, T, H, K, True)
    topk, w = make_routing(T, E, K)
    with pytest.raises(deep_ep._C.EPException, match='kUbAlign'):
        bufs[0].dispatch(make_tokens(T, H).to(DEV), topk_idx=topk.to(DEV), topk_weights=w.to(DEV), num_experts=E,
                         num_max_tokens_per_rank=T, do_expand=True, fused_fp8_quant=True,
                         async_with_compute_stream=True, defer_epilogue=True)
    # one partition never materialises packed rows: the same shape is fine there
    single = deep_ep.EPBuffer(deep_ep.LocalGroup(), num_max_tokens_per_rank=T, hidden=H, num_topk=K,
                              use_fp8_dispatch=True, explicitly_destroy=True)
    (qx, qs), _, _, _, _ = single.dispatch(make_tokens(T, H).to(DEV), topk_idx=topk.to(DEV), num_experts=E,
                                           do_expand=True, fused_fp8_quant=True)
    torch.cuda.synchronize()
    assert qx.size(1) == H and qs.size(1) == 2
    single.destroy()
    for b in bufs:
        b.destroy()


def test_owner_side_whole_rows_shorter_than_a_wave_carry_all_their_weights():
    """From 16384 metadata rows on the owner-side reduce takes whole rows per wave, and a row with a single local
    slot is copied verbatim.  With rows of fewer 16-byte vectors than top-k positions (hidden 64, top-16) the
    weight vector of such a row is wider than its payload: every position of it must still be written."""
    R, max_tokens, H, E, K, A = 2, 8400, 64, 32, 16, 8
    bufs = make_node(R, max_tokens, H, K, False)
    Ts = [max_tokens, max_tokens - 100]
    xs = [make_tokens(T, H, seed=50 + r) for r, T in enumerate(Ts)]
    routing = [make_routing(T, E, K, seed=60 + r, masked=0.85) for r, T in enumerate(Ts)]     # mostly one local slot a row
    topks, ws = [t for t, _ in routing], [w for _, w in routing]
    rows = [bf16_bits(x).view(np.uint8).reshape(x.size(0), -1) for x in xs]
    _, want = oracle_dispatch(rows, [None] * R, [t.numpy() for t in topks], [w.numpy() for w in ws], E, R, A, max_tokens)
    outs = dispatch_all(bufs, [x.to(DEV) for x in xs], [t.to(DEV) for t in topks], [w.to(DEV) for w in ws],
                        num_experts=E, num_max_tokens_per_rank=max_tokens, expert_alignment=A, do_expand=True,
                        do_zero_padding=True, do_cpu_sync=False)
    torch.cuda.synchronize()
    handles = [o[3] for o in outs]
    assert all(h.recv_src_metadata.size(0) >= 16384 for h in handles)          # the whole-row path is the one that runs
    single = sum(int(((want[r]['lay']['recv_src_metadata'][:, :K] >= 0).sum(axis=1) == 1).sum()) for r in range(R))
    assert single > 1000                                                       # and verbatim rows are many
    g = torch.Generator().manual_seed(7)
    ys = [torch.randn((outs[r][0].size(0), H), generator=g).to(torch.bfloat16) for r in range(R)]
    # the combine buffers hold what earlier phases left: poison them, so that a position nobody writes shows
    for b in bufs:
        b.runtime.buffer_tensor().fill_(0x5A)
    res = combine_all(bufs, [y.to(DEV) for y in ys], handles, [o[2] for o in outs], [None] * R)
    torch.cuda.synchronize()
    parts, wvecs = {}, {}
    for r in range(R):
        ne = want[r]['lay']['num_expanded_tokens']
        p, wv = O.combine_partial(ys[r][:ne], torch.from_numpy(want[r]['w']), want[r]['lay']['recv_src_metadata'], R, r, max_tokens)
        parts.update(p)
        wvecs.update(wv)
    for s in range(R):
        ox, ow = O.combine_final(topks[s].numpy(), E, R, s, max_tokens, lambda k: parts[k], lambda k: wvecs[k],
                                 None, None, H, True)
        cx, cw = res[s]
        assert np.array_equal(bf16_bits(cx), bf16_bits(ox)), s
        assert torch.equal(cw.cpu(), ow) and torch.equal(cw.cpu(), ws[s]), s
    for b in bufs:
        b.destroy()
