"""Dispatch (device-side counts, no host sync) + combine recorded into a HIP graph and replayed.

The launches of the library are plain kernel launches on the stream they are given: no allocation,
no memset, no synchronisation, so a decode loop can record them once and replay them.  Every
replay is compared with the eager result on the same inputs, with eager work and synchronisations
between the replays.
"""
import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_routing, make_tokens
from oracle import ep_oracle as O

pytestmark = pytest.mark.gpu
DEV = 'cuda'


@pytest.mark.parametrize('fused_fp8', [False, True])
def test_graph_replay_matches_eager(fused_fp8):
    import deep_ep
    T, H, E, K, A = 128, 1024, 32, 4, 16
    buf = deep_ep.EPBuffer(deep_ep.LocalGroup(0, 1), num_max_tokens_per_rank=T, hidden=H, num_topk=K,
                           use_fp8_dispatch=fused_fp8, explicitly_destroy=True)
    x = torch.empty((T, H), dtype=torch.bfloat16, device=DEV)
    topk = torch.empty((T, K), dtype=torch.int64, device=DEV)
    w = torch.empty((T, K), dtype=torch.float32, device=DEV)
    n_exp = O.no_sync_sizes(1, T, K, E, A)[1]
    y = torch.empty((n_exp, H), dtype=torch.bfloat16, device=DEV)

    def load(seed):
        xs = make_tokens(T, H, seed=seed, outliers=True)
        ts, ws = make_routing(T, E, K, seed=seed, masked=0.2)
        ys = make_tokens(n_exp, H, seed=seed + 100)
        x.copy_(xs), topk.copy_(ts), w.copy_(ws), y.copy_(ys)
        return xs, ts, ws, ys

    def step():
        recv, _, rw, handle, _ = buf.dispatch(x, topk_idx=topk, topk_weights=w, num_experts=E,
                                              num_max_tokens_per_rank=T, expert_alignment=A, do_expand=True,
                                              do_zero_padding=True, do_cpu_sync=False, fused_fp8_quant=fused_fp8)
        cx, cw, _ = buf.combine(y, handle, topk_weights=rw)
        return recv, rw, handle, cx, cw

    load(1)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):              # warm up off the default stream, as torch asks before a capture
        step()
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_recv, g_rw, g_handle, g_cx, g_cw = step()

    for seed in (2, 3, 4, 2):
        xs, ts, ws, ys = load(seed)
        graph.replay()
        torch.cuda.synchronize()
        lay = O.rank_share_layout(ts.numpy(), E, 1, 0, A, T)
        ne = lay['num_expanded_tokens']
        assert np.array_equal(g_handle.recv_src_metadata.cpu().numpy()[:lay['num_recv_tokens']],
                              lay['recv_src_metadata'])
        assert np.array_equal(g_handle.psum_num_recv_tokens_per_expert.cpu().numpy(),
                              lay['psum_num_recv_tokens_per_expert'])
        if fused_fp8:
            q, s = O.quantise(xs)
            eq, es, ew = O.rank_share_dispatch(q.numpy(), s.numpy().view(np.uint32), ws.numpy(), lay)
            assert np.array_equal(g_recv[0].view(torch.uint8).cpu().numpy()[:ne], eq)
            assert np.array_equal(g_recv[1].cpu().numpy().view(np.uint32)[:ne], es)
        else:
            ex, _, ew = O.rank_share_dispatch(bf16_bits(xs), None, ws.numpy(), lay)
            assert np.array_equal(bf16_bits(g_recv)[:ne], ex)
        assert np.array_equal(g_rw.cpu().numpy().view(np.uint32)[:ne], ew.view(np.uint32))
        ox, ow = O.combine_fast(ys, torch.from_numpy(ew), lay['recv_src_metadata'], T, K)
        assert np.array_equal(bf16_bits(g_cx), bf16_bits(ox))
        assert torch.equal(g_cw.cpu(), ow)

        # the same inputs through the eager path, then more eager work before the next replay
        e_recv, e_rw, e_handle, e_cx, e_cw = step()
        torch.cuda.synchronize()
        assert torch.equal(e_cx.view(torch.int16), g_cx.view(torch.int16)) and torch.equal(e_cw, g_cw)
        nr = lay['num_recv_tokens']                      # rows past the received count are not written
        assert torch.equal(e_handle.recv_src_metadata[:nr], g_handle.recv_src_metadata[:nr])
    buf.destroy()
