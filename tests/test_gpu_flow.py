"""The dispatch -> combine -> cached replay flow, checked the way the reference checks itself
(tests/ep/test_ep.py:82-388): not against a fixed layout but through the properties any valid
layout has -- every (token, selection) owns exactly one expanded slot inside its expert's aligned
block, slots of an expert are dense, padding is bitwise zero, the metadata names the source token
and its last local selection -- and through the round trip back to token order.  Expected values
are computed here with plain torch ops on the GPU tensors, independently of the oracle module.
"""
import itertools

import pytest
import torch

from helpers import make_routing, make_tokens

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def _deep_ep():
    import deep_ep
    return deep_ep


def _align(a, b):
    return (a + b - 1) // b * b


def launch(buffer, name, defer_epilogue, **params):
    """As tests/ep/test_ep.py:33-44: the deferred form returns only the event, whose wait runs the
    epilogue and hands back the results."""
    result = getattr(buffer, name)(defer_epilogue=defer_epilogue, **params)
    if defer_epilogue:
        event = result
        return *event.current_stream_wait(release_handle=True), event
    result[-1].current_stream_wait(release_handle=True)
    return result


def dispatch_modes():
    # tests/ep/test_ep.py:25-30
    for alignment, fp8, num_bias in itertools.product((128, 1), (True, False), (0, 1, 2)):
        for col_major in ((False, True) if fp8 else (False,)):
            yield alignment, num_bias, fp8, col_major


def ordered_sum(rows_f32):
    acc = None
    for r in rows_f32:
        acc = r.clone() if acc is None else acc + r
    return acc


def expected_combine(y3, topk_idx, bias):
    """Single partition: one BF16 partial per token (fp32 sum of its selections in ascending
    position), then biases and partial summed in fp32 and rounded once
    (deep_ep/utils/refs.py:155-250 with reduce_in_local=True)."""
    T, K, H = y3.shape
    valid = topk_idx >= 0
    acc = torch.zeros((T, H), dtype=torch.float32, device=y3.device)
    for j in range(K):
        acc = acc + torch.where(valid[:, j:j + 1], y3[:, j].float(), torch.zeros_like(acc))
    partial = acc.to(torch.bfloat16)
    biases = [] if bias is None else ([bias] if isinstance(bias, torch.Tensor) else list(bias))
    if not biases:
        return partial
    total = ordered_sum([b.float() for b in biases]) + partial.float()
    return total.to(torch.bfloat16)


@pytest.mark.parametrize('do_cpu_sync,defer_epilogue', [(True, 0), (False, 0), (True, 1)])
@pytest.mark.parametrize('masked', [0.0, 0.25])
def test_dispatch_combine_flow(do_cpu_sync, defer_epilogue, masked):
    de = _deep_ep()
    max_tokens, T, H, E, K = 192, 181, 512, 16, 4
    buf = de.EPBuffer(de.LocalGroup(0, 1), num_max_tokens_per_rank=max_tokens, hidden=H, num_topk=K,
                      use_fp8_dispatch=False, explicitly_destroy=True, deterministic=True)
    num_cores = buf.get_theoretical_num_sms(E, K)
    topk_cpu, w_cpu = make_routing(T, E, K, seed=11, masked=masked)
    topk_idx, topk_weights = topk_cpu.to(DEV), w_cpu.to(DEV)

    for alignment, num_bias, fp8, col_major in dispatch_modes():
        x = make_tokens(T, H, seed=alignment + num_bias).to(DEV)
        if fp8:
            x_data, sf = de.utils.math.per_token_cast_to_fp8(x)
            sf = sf.view(torch.int16)
            P = sf.size(1)
            if col_major:
                store = torch.empty((T * P,), dtype=torch.int16, device=DEV)
                sf_in = torch.as_strided(store, (T, P), (1, T))
                sf_in.copy_(sf)
            else:
                sf_in = sf
            x_arg, ref_rows, ref_sf = (x_data, sf_in), x_data.view(torch.uint8), sf
        else:
            x_arg, ref_rows, ref_sf = x, x, None
        g = torch.Generator(device=DEV).manual_seed(num_bias)
        bias = None
        if num_bias == 1:
            bias = torch.randn((T, H), device=DEV, generator=g).to(torch.bfloat16)
        elif num_bias == 2:
            bias = tuple(torch.randn((T, H), device=DEV, generator=g).to(torch.bfloat16) for _ in range(2))

        stats = torch.zeros((E,), dtype=torch.int32, device=DEV)
        dispatch_args = dict(x=x_arg, topk_idx=topk_idx, topk_weights=topk_weights, num_sms=0,
                             num_max_tokens_per_rank=max_tokens, num_experts=E, expert_alignment=alignment,
                             async_with_compute_stream=True, do_handle_copy=False, do_cpu_sync=do_cpu_sync,
                             do_expand=True, do_zero_padding=True, use_tma_aligned_col_major_sf=col_major)
        recv_x, recv_idx, recv_w, handle, _ = launch(buf, 'dispatch', defer_epilogue,
                                                     cumulative_local_expert_recv_stats=stats, **dispatch_args)
        torch.cuda.synchronize()
        cached_args = dict(dispatch_args, handle=handle, num_sms=0, do_cpu_sync=False)
        del cached_args['topk_idx']

        recv_data, recv_sf = recv_x if fp8 else (recv_x, None)
        check_x = recv_data.view(torch.uint8) if fp8 else recv_data
        if fp8:
            assert recv_sf.stride() == ((1, recv_data.size(0)) if col_major else (P, 1))

        n_recv = handle.psum_num_recv_tokens_per_rank[-1].item()
        n_exp = _align(handle.psum_num_recv_tokens_per_expert[-1].item(), alignment)
        want_recv = n_recv if do_cpu_sync else max_tokens
        assert handle.num_recv_tokens == want_recv and handle.recv_src_metadata.size(0) == want_recv
        assert recv_idx is None and recv_w is not None
        meta = handle.recv_src_metadata[:n_recv]
        src, slots, master = meta[:, -2].long(), meta[:, :-2], meta[:, -1]

        # received tokens = tokens with at least one selection, each exactly once
        has_any = (topk_idx >= 0).any(dim=1)
        assert n_recv == int(has_any.sum())
        assert torch.equal(torch.sort(src).values, has_any.nonzero().flatten())
        # a slot exactly where the token selected an expert
        valid = slots >= 0
        assert torch.equal(valid, topk_idx[src] >= 0)
        flat = slots[valid].long()
        assert flat.numel() == handle.num_unaligned_recv_tokens_per_expert.sum().item()
        if flat.numel():
            assert flat.min().item() >= 0 and flat.max().item() < n_exp
            assert torch.unique(flat).numel() == flat.numel()
            rows = ref_rows[src].unsqueeze(1).expand(-1, K, -1)[valid]
            assert torch.equal(check_x[flat], rows)
            if fp8:
                assert torch.equal(recv_sf[flat], ref_sf[src].unsqueeze(1).expand(-1, K, -1)[valid])
            assert torch.equal(recv_w[flat], topk_weights[src][valid])
        # last local selection
        pos = torch.arange(K, device=DEV, dtype=meta.dtype).view(1, K)
        assert torch.equal(master, torch.where(valid, pos, torch.full_like(slots, -1)).max(dim=1).values)

        # per-expert blocks: dense, aligned, zero padded; counters
        psum = [0] + handle.psum_num_recv_tokens_per_expert.tolist()
        sel = topk_idx[src]
        for e in range(E):
            start, end = _align(psum[e], alignment), psum[e + 1]
            count = int((topk_idx == e).sum())
            assert end - start == count
            assert stats[e].item() == count and handle.num_unaligned_recv_tokens_per_expert[e].item() == count
            if do_cpu_sync:
                assert handle.num_recv_tokens_per_expert_list[e] == _align(count, alignment)
            mine = torch.sort(slots[sel == e]).values
            assert torch.equal(mine, torch.arange(start, end, device=DEV, dtype=mine.dtype))
            pad_end = _align(end, alignment)
            assert torch.count_nonzero(recv_data[end:pad_end].view(torch.uint8)).item() == 0
            if fp8:
                assert torch.count_nonzero(recv_sf[end:pad_end]).item() == 0
            assert torch.count_nonzero(recv_w[end:pad_end]).item() == 0

        # the same layout twice (deterministic mode, tests/ep/test_ep.py:226-254)
        again_x, _, again_w, again_handle, _ = launch(buf, 'dispatch', defer_epilogue, **dispatch_args)
        torch.cuda.synchronize()
        again_data = again_x[0] if fp8 else again_x
        assert torch.equal(again_handle.recv_src_metadata[:n_recv], meta)
        assert torch.equal(again_data.view(torch.uint8)[:n_exp], recv_data.view(torch.uint8)[:n_exp])
        assert torch.equal(again_w[:n_exp], recv_w[:n_exp])

        # combine: expert output of (token, j) placed at its slot, everything else garbage
        y3 = torch.randn((T, K, H), device=DEV, generator=g).to(torch.bfloat16)
        y = torch.randn((recv_data.size(0), H), device=DEV, generator=g).to(torch.bfloat16) * 100
        if flat.numel():
            y[flat] = y3[src].reshape(n_recv, K, H)[valid]
        want = expected_combine(y3, topk_idx, bias)
        cx, cw, _ = launch(buf, 'combine', defer_epilogue, x=y, handle=handle, topk_weights=recv_w, bias=bias,
                           num_sms=num_cores, async_with_compute_stream=True)
        torch.cuda.synchronize()
        assert torch.equal(cx.view(torch.int16), want.view(torch.int16))
        assert torch.equal(cw, topk_weights)
        if num_bias == 0 and not col_major:
            cx2, cw2, _ = launch(buf, 'combine', defer_epilogue, x=y, handle=handle, bias=bias, num_sms=num_cores,
                                 async_with_compute_stream=True)
            torch.cuda.synchronize()
            assert torch.equal(cx2.view(torch.int16), want.view(torch.int16)) and cw2 is None

        # cached replays after the workspace has been reused (tests/ep/test_ep.py:321-388)
        kept = (handle.psum_num_recv_tokens_per_rank, handle.psum_num_recv_tokens_per_expert,
                handle.num_unaligned_recv_tokens_per_expert, handle.recv_src_metadata,
                handle.dst_buffer_slot_idx, handle.dst_gsge_idx)
        copies = [t.clone() for t in kept]
        pad_mask = torch.ones(n_exp, dtype=torch.bool, device=DEV)
        pad_mask[flat] = False
        for send_weights in (True, False):
            x2 = torch.randn((T, H), device=DEV, generator=g).to(torch.bfloat16) * (8 if send_weights else 0.125)
            if fp8:
                x2_data, sf2 = de.utils.math.per_token_cast_to_fp8(x2)
                sf2 = sf2.view(torch.int16)
                x2_arg = (x2_data, sf2.t().contiguous().t() if col_major else sf2)
                ref2, ref2_sf = x2_data.view(torch.uint8), sf2
            else:
                x2_arg, ref2, ref2_sf = x2, x2, None
            w2 = torch.randn((T, K), device=DEV, generator=g).masked_fill_(topk_idx < 0, 0)
            c_x, c_idx, c_w, c_handle, _ = launch(
                buf, 'dispatch', defer_epilogue,
                **dict(cached_args, x=x2_arg, num_sms=0 if send_weights else handle.num_sms + 1,
                       topk_weights=w2 if send_weights else None))
            torch.cuda.synchronize()
            assert c_handle is handle and c_idx is None and handle.num_sms == num_cores
            for t, saved in zip(kept, copies):
                assert torch.equal(t, saved)
            c_data, c_sf = c_x if fp8 else (c_x, None)
            c_check = c_data.view(torch.uint8) if fp8 else c_data
            if flat.numel():
                assert torch.equal(c_check[flat], ref2[src].unsqueeze(1).expand(-1, K, -1)[valid])
            assert torch.count_nonzero(c_check[:n_exp][pad_mask]).item() == 0
            if c_sf is not None:
                assert c_sf.stride() == ((1, c_data.size(0)) if col_major else (P, 1))
                if flat.numel():
                    assert torch.equal(c_sf[flat], ref2_sf[src].unsqueeze(1).expand(-1, K, -1)[valid])
                assert torch.count_nonzero(c_sf[:n_exp][pad_mask]).item() == 0
            if send_weights:
                if flat.numel():
                    assert torch.equal(c_w[flat], w2[src][valid])
                assert torch.count_nonzero(c_w[:n_exp][pad_mask]).item() == 0
            else:
                assert c_w is None
            ccx, ccw, _ = launch(buf, 'combine', defer_epilogue, x=y, handle=c_handle, topk_weights=c_w, bias=bias,
                                 num_sms=num_cores, async_with_compute_stream=True)
            torch.cuda.synchronize()
            assert torch.equal(ccx.view(torch.int16), want.view(torch.int16))
            if send_weights:
                assert torch.equal(ccw, w2)
            else:
                assert ccw is None
    buf.destroy()


@pytest.mark.parametrize('R', [2, 4])
def test_node_flow(R):
    """The same properties with every rank of the group present (a node of R partitions on this GPU), ragged
    token counts `max(1, N - rank)` as tests/ep/test_ep.py:53: what each partition receives is checked against
    the tokens the *other* partitions hold, and the combine against sums over all partitions' experts."""
    de = _deep_ep()
    max_tokens, H, E, K = 120, 256, 16, 4
    El = E // R
    node = de.LocalNode(R)
    bufs = [de.EPBuffer(node.group(r), num_max_tokens_per_rank=max_tokens, hidden=H, num_topk=K,
                        use_fp8_dispatch=True, explicitly_destroy=True) for r in range(R)]
    Ts = [max(1, max_tokens - r) for r in range(R)]
    routing = [make_routing(T, E, K, seed=40 + r, masked=0.2) for r, T in enumerate(Ts)]
    topk = [t.to(DEV) for t, _ in routing]
    wts = [w.to(DEV) for _, w in routing]

    for alignment, num_bias, fp8, col_major in dispatch_modes():
        if num_bias == 1:
            continue
        g = torch.Generator(device=DEV).manual_seed(alignment + num_bias)
        xs = [torch.randn((T, H), device=DEV, generator=g).to(torch.bfloat16) for T in Ts]
        if fp8:
            pairs = [de.utils.math.per_token_cast_to_fp8(x) for x in xs]
            x_args = [(q, s.view(torch.int16)) for q, s in pairs]
            ref_rows = [q.view(torch.uint8) for q, _ in pairs]
            ref_sfs = [s.view(torch.int16) for _, s in pairs]
        else:
            x_args, ref_rows, ref_sfs = xs, xs, [None] * R
        biases = [tuple(torch.randn((T, H), device=DEV, generator=g).to(torch.bfloat16) for _ in range(2))
                  if num_bias else None for T in Ts]

        events = [bufs[r].dispatch(x_args[r], topk_idx=topk[r], topk_weights=wts[r], num_experts=E,
                                   num_max_tokens_per_rank=max_tokens, expert_alignment=alignment, do_expand=True,
                                   do_zero_padding=True, use_tma_aligned_col_major_sf=col_major,
                                   async_with_compute_stream=True, defer_epilogue=True) for r in range(R)]
        outs = [ev.current_stream_wait(release_handle=True) for ev in events]
        torch.cuda.synchronize()

        y3 = [torch.randn((T, K, H), device=DEV, generator=g).to(torch.bfloat16) for T in Ts]   # expert outputs
        ys = []
        for d, (recv, _, rw, handle) in enumerate(outs):
            recv_data, recv_sf = recv if fp8 else (recv, None)
            check_x = recv_data.view(torch.uint8) if fp8 else recv_data
            n_exp = recv_data.size(0)
            meta = handle.recv_src_metadata
            src, slots, master = meta[:, -2].long(), meta[:, :-2], meta[:, -1]
            src_rank, src_tok = src // max_tokens, src % max_tokens
            # per source: its tokens with a selection on partition d, each once, sources in rank order
            psum = [0] + handle.psum_num_recv_tokens_per_rank.tolist()
            for s in range(R):
                local = (topk[s] >= d * El) & (topk[s] < (d + 1) * El)
                part = slice(psum[s], psum[s + 1])
                assert torch.equal(src_rank[part], torch.full_like(src_rank[part], s))
                assert torch.equal(torch.sort(src_tok[part]).values, local.any(dim=1).nonzero().flatten())
            all_topk = torch.cat([torch.nn.functional.pad(t, (0, 0, 0, max_tokens - t.size(0)), value=-1) for t in topk])
            sel = all_topk[src]                                         # global expert ids of every received row
            local = (sel >= d * El) & (sel < (d + 1) * El)
            assert torch.equal(slots >= 0, local)
            flat = slots[local].long()
            assert flat.numel() == handle.num_unaligned_recv_tokens_per_expert.sum().item()
            assert torch.unique(flat).numel() == flat.numel() and (flat.numel() == 0 or flat.max().item() < n_exp)
            all_rows = torch.cat([torch.nn.functional.pad(r_, (0, 0, 0, max_tokens - r_.size(0))) for r_ in ref_rows])
            assert torch.equal(check_x[flat], all_rows[src].unsqueeze(1).expand(-1, K, -1)[local])
            if fp8:
                assert recv_sf.stride() == ((1, n_exp) if col_major else (recv_sf.size(1), 1))
                all_sf = torch.cat([torch.nn.functional.pad(s_, (0, 0, 0, max_tokens - s_.size(0))) for s_ in ref_sfs])
                assert torch.equal(recv_sf[flat], all_sf[src].unsqueeze(1).expand(-1, K, -1)[local])
            all_w = torch.cat([torch.nn.functional.pad(w_, (0, 0, 0, max_tokens - w_.size(0))) for w_ in wts])
            assert torch.equal(rw[flat], all_w[src][local])
            pos = torch.arange(K, device=DEV, dtype=meta.dtype).view(1, K)
            assert torch.equal(master, torch.where(local, pos, torch.full_like(slots, -1)).max(dim=1).values)
            pe = [0] + handle.psum_num_recv_tokens_per_expert.tolist()
            for e in range(El):
                start, end = _align(pe[e], alignment), pe[e + 1]
                assert end - start == sum(int((t == d * El + e).sum()) for t in topk)
                mine = torch.sort(slots[sel == d * El + e]).values
                assert torch.equal(mine, torch.arange(start, end, device=DEV, dtype=mine.dtype))
                assert torch.count_nonzero(recv_data[end:_align(end, alignment)].view(torch.uint8)).item() == 0
            # expert output of (source token, j) at its slot, garbage elsewhere
            y = torch.randn((n_exp, H), device=DEV, generator=g).to(torch.bfloat16) * 100
            all_y3 = torch.cat([torch.nn.functional.pad(v, (0, 0, 0, 0, 0, max_tokens - v.size(0))) for v in y3])
            if flat.numel():
                y[flat] = all_y3[src][local]
            ys.append(y)

        cevs = [bufs[r].combine(ys[r], outs[r][3], topk_weights=outs[r][2], bias=biases[r],
                                async_with_compute_stream=True, defer_epilogue=True) for r in range(R)]
        res = [ev.current_stream_wait(release_handle=True) for ev in cevs]
        torch.cuda.synchronize()
        for s in range(R):
            # one BF16 partial per destination partition (fp32 sum in ascending position), then biases and
            # partials in ascending position of each partition's last selection (refs.py:175-250)
            T = Ts[s]
            rank_of = torch.where(topk[s] >= 0, topk[s] // El, torch.full_like(topk[s], -1))
            partial = torch.zeros((T, K, H), dtype=torch.float32, device=DEV)        # indexed by master position
            is_master = torch.zeros((T, K), dtype=torch.bool, device=DEV)
            for j in range(K):
                later_same = torch.zeros(T, dtype=torch.bool, device=DEV)
                for jj in range(j + 1, K):
                    later_same |= (rank_of[:, jj] == rank_of[:, j])
                is_master[:, j] = (rank_of[:, j] >= 0) & ~later_same
                acc = torch.zeros((T, H), dtype=torch.float32, device=DEV)
                for jj in range(j + 1):
                    same = (rank_of[:, jj] == rank_of[:, j]) & (rank_of[:, j] >= 0)
                    acc = acc + torch.where(same.unsqueeze(1), y3[s][:, jj].float(), torch.zeros_like(acc))
                partial[:, j] = acc.to(torch.bfloat16).float()
            total = torch.zeros((T, H), dtype=torch.float32, device=DEV)
            if biases[s] is not None:
                total = biases[s][0].float() + biases[s][1].float()
            for j in range(K):
                total = total + torch.where(is_master[:, j:j + 1], partial[:, j], torch.zeros_like(total))
            want = total.to(torch.bfloat16)
            cx, cw = res[s]
            same = (cx.view(torch.int16) == want.view(torch.int16)) | ((cx == 0) & (want == 0))   # sign of zero
            assert bool(same.all()), (alignment, num_bias, fp8, col_major, s)
            assert torch.equal(cw, wts[s])
    for b in bufs:
        b.destroy()
