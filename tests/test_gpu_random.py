"""Seeded random configurations (shapes that are not round numbers, hidden sizes down to one 16-byte
vector and such that a quantised row is not a multiple of 16 bytes, few tokens per expert, many masked
selections, odd top-k) through the single-partition path and through nodes of 2-5 partitions, compared
bit for bit with the oracle."""
import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_routing, make_tokens
from oracle import ep_oracle as O
from test_gpu_node import make_node, oracle_dispatch

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def _configs(n, seed, with_ranks):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        R = int(rng.integers(2, 6)) if with_ranks else 1
        El = int(rng.choice([1, 2, 3, 5, 8, 17]))
        E = R * El
        K = int(min(E, rng.choice([1, 2, 3, 5, 6, 7, 8, 11, 16])))
        H = int(rng.choice([8, 16, 32, 128, 144, 520, 528, 1008, 1024, 2064]))
        T = int(rng.choice([1, 2, 63, 64, 65, 129, 200, 257, 300, 1000]))
        A = int(rng.choice([1, 2, 7, 16, 128]))
        masked = float(rng.choice([0.0, 0.1, 0.5, 0.9]))
        out.append((R, T, H, E, K, A, masked))
    return out


@pytest.mark.parametrize('R,T,H,E,K,A,masked', _configs(60, 1, False))
def test_random_single_partition(R, T, H, E, K, A, masked):
    import deep_ep
    x = make_tokens(T, H, seed=T + H + K, outliers=True)
    topk, w = make_routing(T, E, K, seed=T + E + K, masked=masked)
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    # sized for the BF16 dispatch below, the larger of the two
    buf = deep_ep.EPBuffer(deep_ep.LocalGroup(), num_max_tokens_per_rank=T, hidden=H, num_topk=K, use_fp8_dispatch=False,
                           explicitly_destroy=True)
    kw = dict(topk_idx=topk.to(DEV), topk_weights=w.to(DEV), num_experts=E, num_max_tokens_per_rank=T,
              expert_alignment=A, do_expand=True, do_zero_padding=True)
    rx, _, rw, handle, _ = buf.dispatch(x.to(DEV), **kw)
    (qx, qs), _, _, h2, _ = buf.dispatch(x.to(DEV), fused_fp8_quant=True, **kw)
    torch.cuda.synchronize()
    for h in (handle, h2):
        assert np.array_equal(h.recv_src_metadata.cpu().numpy(), lay['recv_src_metadata'])
        assert np.array_equal(h.psum_num_recv_tokens_per_expert.cpu().numpy(), lay['psum_num_recv_tokens_per_expert'])
        assert np.array_equal(h.dst_buffer_slot_idx.cpu().numpy(), lay['dst_buffer_slot_idx'])
    ex, _, ew = O.rank_share_dispatch(bf16_bits(x), None, w.numpy(), lay)
    assert np.array_equal(bf16_bits(rx), ex)
    assert np.array_equal(rw.cpu().numpy().view(np.uint32), ew.view(np.uint32))
    q, s = O.quantise(x)
    eq, es, _ = O.rank_share_dispatch(q.numpy(), s.numpy().view(np.uint32), w.numpy(), lay)
    assert np.array_equal(qx.view(torch.uint8).cpu().numpy(), eq)
    assert np.array_equal(qs.cpu().numpy().view(np.uint32), es)
    g = torch.Generator().manual_seed(T)
    y = torch.randn((lay['num_expanded_tokens'], H), generator=g).to(torch.bfloat16)
    bias = torch.randn((T, H), generator=g).to(torch.bfloat16)
    cx, cw, _ = buf.combine(y.to(DEV), handle, topk_weights=rw, bias=bias.to(DEV))
    torch.cuda.synchronize()
    ox, ow = O.combine_fast(y, torch.from_numpy(ew), lay['recv_src_metadata'], T, K, bias)
    assert np.array_equal(bf16_bits(cx), bf16_bits(ox))
    assert torch.equal(cw.cpu(), ow)
    buf.destroy()


@pytest.mark.parametrize('R,T,H,E,K,A,masked', _configs(40, 2, True))
def test_random_node(R, T, H, E, K, A, masked):
    bufs = make_node(R, T, H, K, False)
    Ts = [max(1, T - 3 * r) for r in range(R)]
    xs = [make_tokens(n, H, seed=n + r) for r, n in enumerate(Ts)]
    routing = [make_routing(n, E, K, seed=n + 7 * r, masked=masked) for r, n in enumerate(Ts)]
    topks, ws = [t for t, _ in routing], [w for _, w in routing]
    rows = [bf16_bits(x).view(np.uint8).reshape(x.size(0), H * 2) for x in xs]
    sends, want = oracle_dispatch(rows, [None] * R, [t.numpy() for t in topks], [w.numpy() for w in ws], E, R, A, T)
    events = [bufs[r].dispatch(xs[r].to(DEV), topk_idx=topks[r].to(DEV), topk_weights=ws[r].to(DEV), num_experts=E,
                               num_max_tokens_per_rank=T, expert_alignment=A, do_expand=True, do_zero_padding=True,
                               async_with_compute_stream=True, defer_epilogue=True) for r in range(R)]
    outs = [ev.current_stream_wait() for ev in events]
    torch.cuda.synchronize()
    for r, (rx, _, rw, handle) in enumerate(outs):
        lay = want[r]['lay']
        assert np.array_equal(handle.dst_buffer_slot_idx.cpu().numpy(), sends[r][0])
        assert np.array_equal(handle.recv_src_metadata.cpu().numpy(), lay['recv_src_metadata'])
        assert np.array_equal(handle.psum_num_recv_tokens_per_rank.cpu().numpy(), lay['psum_num_recv_tokens_per_rank'])
        assert np.array_equal(rx.view(torch.uint8).cpu().numpy().reshape(rx.size(0), H * 2), want[r]['x'])
        assert np.array_equal(rw.cpu().numpy().view(np.uint32), want[r]['w'].view(np.uint32))
    g = torch.Generator().manual_seed(R + T)
    ys = [torch.randn((o[0].size(0), H), generator=g).to(torch.bfloat16) for o in outs]
    cevs = [bufs[r].combine(ys[r].to(DEV), outs[r][3], topk_weights=outs[r][2], async_with_compute_stream=True,
                            defer_epilogue=True) for r in range(R)]
    res = [ev.current_stream_wait() for ev in cevs]
    torch.cuda.synchronize()
    parts, wvecs = {}, {}
    for r in range(R):
        p, wv = O.combine_partial(ys[r], torch.from_numpy(want[r]['w']), want[r]['lay']['recv_src_metadata'], R, r, T)
        parts.update(p)
        wvecs.update(wv)
    for s in range(R):
        ox, ow = O.combine_final(topks[s].numpy(), E, R, s, T, lambda k: parts[k], lambda k: wvecs[k], None, None, H, True)
        assert np.array_equal(bf16_bits(res[s][0]), bf16_bits(ox)), s
        assert torch.equal(res[s][1].cpu(), ow)
    for b in bufs:
        b.destroy()
