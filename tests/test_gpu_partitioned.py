"""One GPU's share of an EP-R layout: R partitions of the arena, this GPU being partition `rank`.
Checks the partition-major packed regions, the expansion of the own region, and the two-level combine
(owner-side partials, token-side final reduce) bit-exactly against the oracle."""
import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_routing, make_tokens
from oracle import ep_oracle as O

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def _buffer(T, H, K, R, rank, fp8=False):
    import deep_ep
    return deep_ep.EPBuffer(deep_ep.LocalGroup(rank, R), num_max_tokens_per_rank=T, hidden=H, num_topk=K,
                            use_fp8_dispatch=fp8, explicitly_destroy=True)


def _regions(buf, R, maxT, token_bytes):
    raw = buf.runtime.buffer_tensor()[:R * maxT * token_bytes].cpu().numpy()
    return raw.reshape(R, maxT, token_bytes)


def check_packed(buf, lay_tok, regions_ref, R, maxT, K, with_sf_bytes):
    got = _regions(buf, R, maxT, lay_tok.num_bytes())
    HB = lay_tok.num_hidden_bytes
    fields = [(0, HB), (lay_tok.topk_idx_offset, lay_tok.topk_idx_offset + 8 * K),
              (lay_tok.topk_weights_offset, lay_tok.topk_weights_offset + 4 * K),
              (lay_tok.src_token_global_idx_offset, lay_tok.src_token_global_idx_offset + 4)]
    if with_sf_bytes:
        fields.append((lay_tok.sf_offset, lay_tok.sf_offset + with_sf_bytes))
    for r in range(R):
        n = regions_ref[r].shape[0]
        for lo, hi in fields:
            assert np.array_equal(got[r, :n, lo:hi], regions_ref[r][:, lo:hi]), (r, lo, hi)


PCASES = [
    # T, H, E, K, A, R, rank, masked
    (64, 256, 8, 2, 1, 2, 0, 0.0),
    (200, 512, 32, 6, 16, 4, 3, 0.15),
    (150, 1024, 64, 8, 128, 32, 17, 0.1),      # R >= K: partial groups are top-k positions
    (130, 512, 12, 6, 8, 3, 1, 0.2),           # R < K: partial groups are partitions
]


@pytest.mark.parametrize('T,H,E,K,A,R,rank,masked', PCASES)
@pytest.mark.parametrize('mode', ['bf16', 'fp8_fused', 'fp8_prequant'])
def test_partitioned_dispatch(T, H, E, K, A, R, rank, masked, mode):
    x = make_tokens(T, H, seed=T + R, outliers=True)
    topk, w = make_routing(T, E, K, seed=T + R, masked=masked)
    lay = O.rank_share_layout(topk.numpy(), E, R, rank, A, T)
    buf = _buffer(T, H, K, R, rank, fp8=mode != 'bf16')
    kw = dict(topk_idx=topk.to(DEV), topk_weights=w.to(DEV), num_experts=E, num_max_tokens_per_rank=T,
              expert_alignment=A, do_expand=True, do_zero_padding=True)
    q, s = O.quantise(x)
    if mode == 'bf16':
        rows, sf_rows, sfb = bf16_bits(x).view(np.uint8).reshape(T, -1), None, 0
        recv, _, rw, handle, _ = buf.dispatch(x.to(DEV), **kw)
        rx, rsf = recv, None
    else:
        rows, sf_rows = q.numpy(), s.numpy().view(np.uint8).reshape(T, -1)
        sfb = sf_rows.shape[1]
        if mode == 'fp8_fused':
            (rx, rsf), _, rw, handle, _ = buf.dispatch(x.to(DEV), fused_fp8_quant=True, **kw)
        else:
            xin = (q.view(torch.float8_e4m3fn).to(DEV), s.view(torch.int16).to(DEV))
            (rx, rsf), _, rw, handle, _ = buf.dispatch(xin, **kw)
    torch.cuda.synchronize()

    # handle tensors
    for name in ('psum_num_recv_tokens_per_rank', 'psum_num_recv_tokens_per_expert',
                 'num_unaligned_recv_tokens_per_expert', 'dst_buffer_slot_idx', 'dst_gsge_idx', 'recv_src_metadata'):
        assert np.array_equal(getattr(handle, name).cpu().numpy(), lay[name]), name
    assert handle.num_recv_tokens == lay['num_recv_tokens']
    assert handle.num_expanded_tokens == lay['num_expanded_tokens']

    # packed partition-major regions (what a transport would ship)
    tok = O.dispatch_token_layout(rows.shape[1], sfb // 2, K)
    ref_regions = O.pack_regions(rows, sf_rows, topk.numpy(), w.numpy(), lay['dst_buffer_slot_idx'],
                                 lay['num_send_tokens_per_rank'], E, R, rank, T)
    check_packed(buf, tok, ref_regions, R, T, K, sfb)

    # expansion of the own region
    ex, es, ew = O.rank_share_dispatch(rows, sf_rows, w.numpy(), lay)
    got_x = rx.view(torch.uint8).cpu().numpy().reshape(rx.size(0), -1)
    assert np.array_equal(got_x, ex)
    if sfb:
        assert np.array_equal(np.ascontiguousarray(rsf.cpu().numpy()).view(np.uint8).reshape(rsf.size(0), -1), es)
    assert np.array_equal(rw.cpu().numpy().view(np.uint32), ew.view(np.uint32))

    # cached replay: new payload and weights through the same layout
    x2 = make_tokens(T, H, seed=T + R + 1)
    w2 = torch.randn((T, K), generator=torch.Generator().manual_seed(3)).masked_fill(topk < 0, 0)
    if mode == 'bf16':
        rows2 = bf16_bits(x2).view(np.uint8).reshape(T, -1)
        r2, _, rw2, h2, _ = buf.dispatch(x2.to(DEV), topk_weights=w2.to(DEV), handle=handle, do_expand=True,
                                         do_zero_padding=True)
        torch.cuda.synchronize()
        assert h2 is handle
        ex2, _, ew2 = O.rank_share_dispatch(rows2, None, w2.numpy(), lay)
        assert np.array_equal(r2.view(torch.uint8).cpu().numpy().reshape(r2.size(0), -1), ex2)
        assert np.array_equal(rw2.cpu().numpy().view(np.uint32), ew2.view(np.uint32))
    buf.destroy()


@pytest.mark.parametrize('T,H,E,K,A,R,rank,masked', PCASES)
@pytest.mark.parametrize('nbias', [0, 2])
def test_partitioned_combine(T, H, E, K, A, R, rank, masked, nbias):
    import deep_ep
    x = make_tokens(T, H, seed=T)
    topk, w = make_routing(T, E, K, seed=T + 2 * R, masked=masked)
    if T > 7:
        topk[7] = -1
        w[7] = 0
    lay = O.rank_share_layout(topk.numpy(), E, R, rank, A, T)
    buf = _buffer(T, H, K, R, rank)
    _, _, rw, handle, _ = buf.dispatch(x.to(DEV), topk_idx=topk.to(DEV), topk_weights=w.to(DEV), num_experts=E,
                                       num_max_tokens_per_rank=T, expert_alignment=A, do_expand=True,
                                       do_zero_padding=True)
    g = torch.Generator().manual_seed(5)
    y = torch.randn((lay['num_expanded_tokens'], H), generator=g).to(torch.bfloat16)
    bias = [torch.randn((T, H), generator=g).to(torch.bfloat16) for _ in range(nbias)]
    tokb = O.combine_token_layout(H, K).num_bytes()
    G = min(K, R)
    epr = E // R

    # what the other partitions' owners would have sent: random partials at the master positions, each with
    # a weight vector that is non-zero only at the positions living on that partition
    other = np.zeros((G * T, tokb), dtype=np.uint8)
    other_p, other_w = {}, {}
    tk = topk.numpy()
    for t in range(T):
        seen = set()
        for j in range(K - 1, -1, -1):
            e = int(tk[t, j])
            if e < 0 or e // epr in seen:
                continue
            r = e // epr
            seen.add(r)
            if r == rank:
                continue
            grp = r if R < K else j
            p = torch.randn(H, generator=g).to(torch.bfloat16)
            wv = torch.zeros(K)
            for jj in range(K):
                if tk[t, jj] >= 0 and tk[t, jj] // epr == r:
                    wv[jj] = w[t, jj]
            key = (grp, rank * T + t)
            other_p[key], other_w[key] = p, wv
            row = other[grp * T + t]
            row[:H * 2] = bf16_bits(p).view(np.uint8)
            row[H * 2:H * 2 + 4 * K] = wv.numpy().view(np.uint8)
    arena = buf.runtime.buffer_tensor()
    arena[:other.size].copy_(torch.from_numpy(other.reshape(-1)).to(DEV))

    b_arg = None if nbias == 0 else tuple(b.to(DEV) for b in bias)
    ev = buf.combine(y.to(DEV), handle, topk_weights=rw, bias=b_arg, async_with_compute_stream=True,
                     defer_epilogue=True)                      # owner-side partials are enqueued here
    torch.cuda.synchronize()
    own_p, own_w = O.combine_partial(y, rw.cpu(), lay['recv_src_metadata'], R, rank, T)
    got = arena[:G * T * tokb].cpu().numpy().reshape(G * T, tokb)
    for (grp, src), p in own_p.items():
        row = got[grp * T + (src - rank * T)]
        assert np.array_equal(row[:H * 2].view(np.uint16), bf16_bits(p)), (grp, src)
        assert np.array_equal(row[H * 2:H * 2 + 4 * K].view(np.float32), own_w[(grp, src)].numpy())
    cx, cw = ev.current_stream_wait()                           # token-side final reduce
    torch.cuda.synchronize()
    parts = dict(other_p)
    parts.update(own_p)
    wvs = dict(other_w)
    wvs.update(own_w)
    ox, ow = O.combine_final(tk, E, R, rank, T, lambda k: parts[k], lambda k: wvs[k],
                             bias[0] if nbias else None, bias[1] if nbias else None, H, True)
    assert np.array_equal(bf16_bits(cx), bf16_bits(ox))
    assert torch.equal(cw.cpu(), ow)
    assert torch.equal(cw.cpu(), w)
    buf.destroy()
