"""Edge cases of the dispatch/combine path: empty and fully masked inputs, ragged sizes, odd top-k and
hidden sizes, stream/lifetime behaviour under allocator reuse, running statistics, handle guards."""
import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_routing, make_tokens
from oracle import ep_oracle as O

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def _buffer(maxT, H, K, R=1, rank=0, **kw):
    import deep_ep
    return deep_ep.EPBuffer(deep_ep.LocalGroup(rank, R), num_max_tokens_per_rank=maxT, hidden=H, num_topk=K,
                            explicitly_destroy=True, **kw)


def _roundtrip(T, maxT, H, E, K, A, topk, w, x, R=1, rank=0, fused=False, seed=0):
    lay = O.rank_share_layout(topk.numpy(), E, R, rank, A, maxT)
    buf = _buffer(maxT, H, K, R, rank, use_fp8_dispatch=fused)
    out = buf.dispatch(x.to(DEV), topk_idx=topk.to(DEV), topk_weights=w.to(DEV), num_experts=E,
                       num_max_tokens_per_rank=maxT, expert_alignment=A, do_expand=True, do_zero_padding=True,
                       fused_fp8_quant=fused)
    recv, _, rw, handle, _ = out
    torch.cuda.synchronize()
    assert np.array_equal(handle.recv_src_metadata.cpu().numpy(), lay['recv_src_metadata'])
    assert np.array_equal(handle.dst_buffer_slot_idx.cpu().numpy(), lay['dst_buffer_slot_idx'])
    assert handle.num_expanded_tokens == lay['num_expanded_tokens']
    if fused:
        q, s = O.quantise(x)
        ex, es, ew = O.rank_share_dispatch(q.numpy(), s.numpy().view(np.uint32), w.numpy(), lay)
        assert np.array_equal(recv[0].view(torch.uint8).cpu().numpy().reshape(ex.shape), ex)
        assert np.array_equal(recv[1].cpu().numpy().view(np.uint32).reshape(es.shape), es)
    else:
        ex, _, ew = O.rank_share_dispatch(bf16_bits(x).reshape(T, H), None, w.numpy(), lay)
        assert np.array_equal(bf16_bits(recv).reshape(ex.shape), ex)
    assert np.array_equal(rw.cpu().numpy().view(np.uint32), ew.view(np.uint32))
    if R == 1:
        y = make_tokens(lay['num_expanded_tokens'], H, seed=seed + 1)
        cx, cw, _ = buf.combine(y.to(DEV), handle, topk_weights=rw)
        torch.cuda.synchronize()
        ox, ow = O.combine_fast(y, torch.from_numpy(ew), lay['recv_src_metadata'], T, K)
        assert np.array_equal(bf16_bits(cx).reshape(T, H), bf16_bits(ox).reshape(T, H))
        assert torch.equal(cw.cpu(), ow)
    buf.destroy()
    return lay


def test_empty_input():
    T, H, E, K = 0, 256, 8, 2
    x = torch.empty((0, H), dtype=torch.bfloat16)
    topk = torch.empty((0, K), dtype=torch.int64)
    w = torch.empty((0, K), dtype=torch.float32)
    lay = _roundtrip(T, 16, H, E, K, 4, topk, w, x)
    assert lay['num_recv_tokens'] == 0 and lay['num_expanded_tokens'] == 0


def test_every_slot_masked():
    T, H, E, K = 40, 256, 8, 3
    x = make_tokens(T, H)
    topk = torch.full((T, K), -1, dtype=torch.int64)
    w = torch.zeros((T, K))
    lay = _roundtrip(T, T, H, E, K, 8, topk, w, x)
    assert lay['num_recv_tokens'] == 0
    # combine of an empty receive stream: bias sum, or zeros
    buf = _buffer(T, H, K)
    _, _, rw, handle, _ = buf.dispatch(x.to(DEV), topk_idx=topk.to(DEV), topk_weights=w.to(DEV), num_experts=E,
                                       expert_alignment=8, do_expand=True)
    y = torch.empty((handle.num_expanded_tokens, H), dtype=torch.bfloat16, device=DEV)
    b0, b1 = make_tokens(T, H, seed=3), make_tokens(T, H, seed=4)
    cx, cw, _ = buf.combine(y, handle, topk_weights=rw)
    assert int(cx.count_nonzero()) == 0 and int(cw.count_nonzero()) == 0
    cx, _, _ = buf.combine(y, handle, bias=b0.to(DEV))
    assert torch.equal(cx.cpu(), b0)
    cx, _, _ = buf.combine(y, handle, bias=(b0.to(DEV), b1.to(DEV)))
    assert torch.equal(cx.cpu(), (b0.float() + b1.float()).to(torch.bfloat16))
    buf.destroy()


@pytest.mark.parametrize('T,maxT,H,E,K,A,masked,fused', [
    (33, 64, 384, 6, 1, 1, 0.0, False),        # top-1, hidden not a multiple of 512
    (100, 100, 1040, 10, 3, 3, 0.2, True),     # odd top-k (generic combine), odd alignment, ragged last group
    (257, 300, 2064, 40, 5, 16, 0.3, True),
    (129, 129, 7168, 256, 7, 128, 0.0, False),
    (5, 4096, 512, 64, 8, 64, 0.0, True),      # far fewer tokens than the buffer allows
    (1000, 1000, 128, 4, 4, 32, 0.0, False),   # every token on every expert
])
def test_ragged_shapes(T, maxT, H, E, K, A, masked, fused):
    x = make_tokens(T, H, seed=T, outliers=True)
    topk, w = make_routing(T, E, K, seed=T, masked=masked)
    _roundtrip(T, maxT, H, E, K, A, topk, w, x, fused=fused, seed=T)


def test_duplicate_experts_in_a_row_are_legal():
    T, H, E, K = 50, 256, 4, 4
    x = make_tokens(T, H)
    topk, w = make_routing(T, E, K, seed=1)
    topk[:, 1] = topk[:, 0]
    topk[::3, 3] = topk[::3, 2]
    _roundtrip(T, T, H, E, K, 4, topk, w, x)
    _roundtrip(T, T, H, E, K, 4, topk, w, x, R=2, rank=1)


def test_current_stream_and_input_lifetime():
    """Everything runs on the caller's current stream; inputs released right after the call stay valid
    for the deferred epilogue even when the allocator hands their memory to someone else."""
    import deep_ep
    T, H, E = 16, 1024, 4
    buf = _buffer(T, H, 1)
    stream = torch.cuda.Stream()
    for defer in (False, True):
        for it in range(2):
            with torch.cuda.stream(stream):
                x = torch.empty((T, H), dtype=torch.bfloat16, device=DEV)
                topk = torch.full((T, 1), it % E, dtype=torch.int64, device=DEV)
                if it:
                    torch.cuda._sleep(50_000_000)
                x.fill_(1 + 10 * it)
                res = buf.dispatch(x, topk_idx=topk, num_experts=E, expert_alignment=1, do_cpu_sync=False,
                                   do_expand=True, async_with_compute_stream=True, defer_epilogue=defer)
                assert torch.cuda.current_stream() == stream
                if defer:
                    ev = res
                else:
                    rx, _, _, handle, ev = res
                    snap = rx[:T].clone()
            del x
            with torch.cuda.stream(stream):
                pressure = torch.full((T, H), -100, dtype=torch.bfloat16, device=DEV)
                if defer:
                    rx, _, _, handle = ev.wait()
                    snap = rx[:T].clone()
                else:
                    ev.wait()
            stream.synchronize()
            assert int(handle.psum_num_recv_tokens_per_rank[-1]) == T
            assert torch.equal(snap, torch.full_like(snap, 1 + 10 * it))
            del pressure
    # events: a hook registered on an EventOverlap runs once, on the waiting stream
    producer, consumer = torch.cuda.Stream(), torch.cuda.Stream()
    src = torch.zeros(4096, device=DEV)
    torch.cuda.synchronize()
    with torch.cuda.stream(producer):
        torch.cuda._sleep(50_000_000)
        src.fill_(3)
        ready = deep_ep.EventHandle()
    with torch.cuda.stream(stream):
        ready.current_stream_wait()
        mid = src * 2
        ev = deep_ep.EventOverlap(deep_ep.EventHandle())
    calls = []
    ev.register_hook_after_wait(lambda: calls.append(torch.cuda.current_stream()) or mid + 1)
    with torch.cuda.stream(consumer):
        out = ev.wait()
        assert ev.wait() is None
    consumer.synchronize()
    assert calls == [consumer] and torch.equal(out, torch.full_like(out, 7))
    buf.destroy()


def test_running_expert_statistics_accumulate():
    T, H, E, K = 120, 256, 16, 4
    x = make_tokens(T, H).to(DEV)
    stats = torch.zeros(E, dtype=torch.int32, device=DEV)
    buf = _buffer(T, H, K)
    total = np.zeros(E, dtype=np.int64)
    for seed in range(3):
        topk, _ = make_routing(T, E, K, seed=seed, masked=0.1)
        buf.dispatch(x, topk_idx=topk.to(DEV), cumulative_local_expert_recv_stats=stats, num_experts=E,
                     do_expand=True)
        total += np.bincount(topk[topk >= 0].numpy(), minlength=E)
    torch.cuda.synchronize()
    assert np.array_equal(stats.cpu().numpy(), total)
    buf.destroy()


def test_handle_guards_topk_idx_against_mutation():
    T, H, E, K = 32, 256, 8, 2
    topk, w = make_routing(T, E, K)
    tg = topk.to(DEV)
    buf = _buffer(T, H, K)
    rx, _, _, handle, _ = buf.dispatch(make_tokens(T, H).to(DEV), topk_idx=tg, num_experts=E, do_expand=True)
    assert handle.topk_idx is tg
    tg[0, 0] = 1
    with pytest.raises(AssertionError, match='must not be modified'):
        buf.combine(rx, handle)
    buf.destroy()


def test_deterministic_flag_gives_the_same_layout():
    T, H, E, K, A = 300, 512, 32, 4, 16
    x = make_tokens(T, H).to(DEV)
    topk, w = make_routing(T, E, K, seed=9, masked=0.1)
    outs = []
    for det in (False, True):
        import deep_ep
        buf = deep_ep.EPBuffer(deep_ep.LocalGroup(), num_max_tokens_per_rank=T, hidden=H, num_topk=K,
                               deterministic=det, explicitly_destroy=True)
        rx, _, rw, h, ev = buf.dispatch(x, topk_idx=topk.to(DEV), topk_weights=w.to(DEV), num_experts=E,
                                        expert_alignment=A, do_expand=True, do_zero_padding=True,
                                        async_with_compute_stream=det)
        if det:
            ev.current_stream_wait()      # the canonicalising hook runs when the event is waited on
        torch.cuda.synchronize()
        outs.append((rx.clone(), rw.clone(), h.recv_src_metadata.clone()))
        if det:
            assert h.cached_recv_src_metadata_before_sort is not None
        buf.destroy()
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    # inside every expert the valid rows ascend with the source token (the reference's sorted order)
    meta = outs[0][2].cpu().numpy()
    for e in range(E):
        tt, jj = np.nonzero(topk.numpy()[meta[:, K]] == e)
        assert np.all(np.diff(meta[tt, jj]) > 0)


@pytest.mark.parametrize('T,E,K,R,rank', [(700, 64, 6, 1, 0), (1500, 256, 8, 8, 3), (300, 2048, 4, 1, 0), (128, 256, 8, 1, 0),
                                         (129, 256, 8, 4, 2), (300, 2048, 8, 1, 0), (300, 2048, 32, 1, 0)])
def test_single_and_multi_block_layouts_agree_with_oracle(T, E, K, R, rank):
    """128 tokens fit one layout block (no counting pass runs); 129 need the counting pass.  2048 experts of one
    partition are more count columns than the slot assignment that sums the counts itself has threads for: the scan
    kernel runs at any size."""
    H, A = 128, 16
    topk, w = make_routing(T, E, K, seed=T, masked=0.1)
    lay = O.rank_share_layout(topk.numpy(), E, R, rank, A, T)
    buf = _buffer(T, H, K, R, rank)
    _, _, _, handle, _ = buf.dispatch(make_tokens(T, H).to(DEV), topk_idx=topk.to(DEV), topk_weights=w.to(DEV),
                                      num_experts=E, expert_alignment=A, do_expand=True)
    torch.cuda.synchronize()
    for name in ('psum_num_recv_tokens_per_rank', 'psum_num_recv_tokens_per_expert',
                 'num_unaligned_recv_tokens_per_expert', 'dst_buffer_slot_idx', 'recv_src_metadata'):
        assert np.array_equal(getattr(handle, name).cpu().numpy(), lay[name]), name
    assert handle.num_recv_tokens_per_expert_list == lay['num_recv_tokens_per_expert_list']
    buf.destroy()


def test_block_counts_at_their_16_bit_bound():
    """Every position of every token names expert 0: each of the 44 layout blocks counts 128 x 32 = 4096 entries for it,
    the most a block can, and one thread of the slot assignment sums all 44 rows of that column (1024 experts: one row
    stripe) in its 16-bit partial sums, 11 rows at a time."""
    T, H, E, K, A = 5632, 128, 1024, 32, 16
    topk = torch.zeros((T, K), dtype=torch.int64)
    topk[::7, 3] = -1
    w = torch.rand((T, K))
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    buf = _buffer(T, H, K)
    _, _, _, handle, _ = buf.dispatch(make_tokens(T, H).to(DEV), topk_idx=topk.to(DEV), topk_weights=w.to(DEV),
                                      num_experts=E, expert_alignment=A, do_expand=True)
    torch.cuda.synchronize()
    for name in ('psum_num_recv_tokens_per_rank', 'psum_num_recv_tokens_per_expert',
                 'num_unaligned_recv_tokens_per_expert', 'dst_buffer_slot_idx', 'recv_src_metadata'):
        assert np.array_equal(getattr(handle, name).cpu().numpy(), lay[name]), name
    buf.destroy()


@pytest.mark.parametrize('T,E,K,R,rank', [(1500, 256, 8, 1, 0), (700, 64, 6, 4, 1), (700, 64, 6, 1, 0), (257, 256, 8, 1, 0),
                                         (1000, 2048, 2, 1, 0), (40000, 64, 2, 8, 3)])
def test_layout_paths_agree(T, E, K, R, rank):
    """Several layout workgroups, four ways to the counts of the workgroups before one: the slot assignment sums the
    histograms itself, or reads the prefixes a scan kernel left, or (one partition, few blocks: the last three shapes) no
    histogram kernel runs and it counts the ids of all blocks itself.  Same handle tensors every way.  (The last shape:
    313 blocks of a partition with 16 count columns, which the slot assignment still sums itself.)"""
    import deep_ep
    H, A = 128, 16
    topk, w = make_routing(T, E, K, seed=T + 1, masked=0.1)
    lay = O.rank_share_layout(topk.numpy(), E, R, rank, A, T)
    try:
        # fold_max 0: every multi-block layout takes the scan kernel; recount limit 0: the histogram kernel always runs
        for fold_max, recount in ((256, 48), (256, 0), (0, 0)):
            deep_ep._C.set_layout_fold_max_blocks(fold_max)
            deep_ep._C.set_layout_recount_limit(recount)
            buf = _buffer(T, H, K, R, rank)
            _, _, _, handle, _ = buf.dispatch(make_tokens(T, H).to(DEV), topk_idx=topk.to(DEV), topk_weights=w.to(DEV),
                                              num_experts=E, expert_alignment=A, do_expand=True)
            torch.cuda.synchronize()
            for name in ('psum_num_recv_tokens_per_rank', 'psum_num_recv_tokens_per_expert',
                         'num_unaligned_recv_tokens_per_expert', 'dst_buffer_slot_idx', 'recv_src_metadata'):
                assert np.array_equal(getattr(handle, name).cpu().numpy(), lay[name]), (fold_max, recount, name)
            buf.destroy()
    finally:
        deep_ep._C.set_layout_fold_max_blocks(256)
        deep_ep._C.set_layout_recount_limit(48)


@pytest.mark.parametrize('fused', [False, True])
def test_exact_sync_sizes_allocate_what_the_results_show(fused):
    """A host-synchronised dispatch returns views of bound-sized storage by default; with `set_exact_sync_sizes()` the
    storage is exactly what the shapes show, and the results are the same bytes."""
    T, H, E, K, A = 777, 512, 32, 4, 64
    topk, w = make_routing(T, E, K, seed=3, masked=0.2)
    x = make_tokens(T, H, seed=3)
    buf = _buffer(T, H, K, use_fp8_dispatch=fused)
    kw = dict(topk_idx=topk.to(DEV), topk_weights=w.to(DEV), num_experts=E, expert_alignment=A, do_expand=True,
              do_zero_padding=True, fused_fp8_quant=fused)
    r0, _, w0, h0, _ = buf.dispatch(x.to(DEV), **kw)
    buf.set_exact_sync_sizes(True)
    r1, _, w1, h1, _ = buf.dispatch(x.to(DEV), **kw)
    buf.set_exact_sync_sizes(False)
    torch.cuda.synchronize()
    p0, p1 = (r0[0], r1[0]) if fused else (r0, r1)
    assert p1.shape == p0.shape and p1.untyped_storage().nbytes() == p1.numel() * p1.element_size()
    assert p0.untyped_storage().nbytes() > p0.numel() * p0.element_size()
    assert w1.untyped_storage().nbytes() == w1.numel() * 4
    assert h1.recv_src_metadata.untyped_storage().nbytes() == h1.recv_src_metadata.numel() * 4
    assert torch.equal(p0.view(torch.uint8), p1.view(torch.uint8)) and torch.equal(w0, w1)
    if fused:
        assert torch.equal(r0[1], r1[1]) and r1[1].untyped_storage().nbytes() == r1[1].numel() * 4
    assert torch.equal(h0.recv_src_metadata, h1.recv_src_metadata)
    assert h0.num_recv_tokens_per_expert_list == h1.num_recv_tokens_per_expert_list
    buf.destroy()


def test_epilogue_of_an_overtaken_dispatch_is_refused():
    """Two deferred dispatches on one buffer: the second launch overwrites the slot map in the buffer's
    workspace, so the first one's copy epilogue must not run any more; the host refuses it."""
    import deep_ep
    T, H, E, K, A = 200, 128, 16, 4, 8
    buf = _buffer(T, H, K)
    x = make_tokens(T, H).to(DEV)
    topk_a, w_a = make_routing(T, E, K, seed=1)
    topk_b, w_b = make_routing(T, E, K, seed=2)
    kw = dict(num_experts=E, expert_alignment=A, do_expand=True, do_zero_padding=True,
              async_with_compute_stream=True, defer_epilogue=True)
    first = buf.dispatch(x, topk_idx=topk_a.to(DEV), topk_weights=w_a.to(DEV), **kw)
    second = buf.dispatch(x, topk_idx=topk_b.to(DEV), topk_weights=w_b.to(DEV), **kw)
    with pytest.raises(deep_ep._C.EPException, match='latest dispatch launch'):
        first.current_stream_wait()
    rx, _, rw, handle = second.current_stream_wait()       # the latest one is served, and correctly
    torch.cuda.synchronize()
    lay = O.rank_share_layout(topk_b.numpy(), E, 1, 0, A, T)
    assert np.array_equal(handle.recv_src_metadata.cpu().numpy(), lay['recv_src_metadata'])
    ex, _, ew = O.rank_share_dispatch(bf16_bits(x.cpu()).view(np.int16), None, w_b.numpy(), lay)
    assert np.array_equal(bf16_bits(rx).view(np.int16), ex)
    buf.destroy()


def test_plain_c_caller_of_the_abi():
    """deep_ep/lib/abi_client (csrc/abi_client.c, built with gcc): the C ABI used without torch or C++,
    with hipMalloc'd tensors and its own stream; it checks the layout and an exact round trip itself."""
    import os
    import subprocess
    import deep_ep
    exe = os.path.join(os.path.dirname(deep_ep.__file__), 'lib', 'abi_client')
    assert os.path.exists(exe), 'run deep_ep/_build.py'
    res = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stderr
    assert res.stdout.startswith('abi_client: ok')


def test_previous_event_orders_the_dispatch_behind_another_stream():
    """The inputs are produced on a side stream; `previous_event` (captured there) is all that orders the
    dispatch on the current stream behind them."""
    import deep_ep
    T, H, E, K = 2048, 2048, 16, 4
    buf = deep_ep.EPBuffer(deep_ep.LocalGroup(), num_max_tokens_per_rank=T, hidden=H, num_topk=K, explicitly_destroy=True)
    topk, w = make_routing(T, E, K, seed=3)
    tg, wg = topk.to(DEV), w.to(DEV)
    src = make_tokens(T, H, seed=3).to(DEV)
    x = torch.zeros_like(src)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for _ in range(20):                       # keep the side stream busy before the inputs appear
            junk = torch.randn((2048, 2048), device=DEV) @ torch.randn((2048, 2048), device=DEV)
        x.copy_(src)
        ready = deep_ep.EPBuffer.capture()
    rx, _, _, handle, _ = buf.dispatch(x, topk_idx=tg, topk_weights=wg, num_experts=E, do_expand=True,
                                       previous_event=ready)
    torch.cuda.synchronize()
    del junk
    meta = handle.recv_src_metadata.long()
    valid = meta[:, :K] >= 0
    assert torch.equal(rx[meta[:, :K][valid]], src[meta[:, K]].unsqueeze(1).expand(-1, K, -1)[valid])
    buf.destroy()


@pytest.mark.parametrize('hw_convert', [True, False])
def test_fused_quantiser_on_non_finite_inputs(hw_convert):
    """inf, -inf, NaN, -NaN, an all-zero row and the largest BF16 go through the fused quantiser exactly as
    through the reference's arithmetic (deep_ep/utils/math.py:30-38: amax and clamp propagate a NaN to the
    whole 128-channel group and its scale; an infinity makes the multiplier zero)."""
    import deep_ep
    T, H, E, K = 8, 256, 4, 1
    x = make_tokens(T, H, seed=12)
    x[0, 3], x[1, 5], x[2, 7], x[5, 130] = float('inf'), float('-inf'), float('nan'), -float('nan')
    x[3, :] = 0
    x[4, 0] = 3.3e38
    topk = torch.zeros((T, K), dtype=torch.int64)
    q, s = O.quantise(x)
    buf = deep_ep.EPBuffer(deep_ep.LocalGroup(), num_max_tokens_per_rank=T, hidden=H, num_topk=K, use_fp8_dispatch=True,
                           explicitly_destroy=True)
    deep_ep._C.set_fp8_hw_convert(hw_convert)
    try:
        (rx, rsf), _, _, _, _ = buf.dispatch(x.to(DEV), topk_idx=topk.to(DEV), num_experts=E, do_expand=True,
                                             fused_fp8_quant=True)
        torch.cuda.synchronize()
    finally:
        deep_ep._C.set_fp8_hw_convert(True)
    assert np.array_equal(rx.view(torch.uint8).cpu().numpy(), q.numpy())
    assert np.array_equal(rsf.cpu().numpy().view(np.uint32), s.numpy().view(np.uint32))
    assert int((q.numpy()[2, :128] == 0x7f).sum()) == 128          # the NaN poisons its whole group
    buf.destroy()


def test_combine_on_non_finite_expert_outputs():
    """inf, -inf (their sum: NaN) and NaN rows go through the fp32 accumulation and the single rounding as in
    the reference's ordered sum (deep_ep/utils/refs.py:155-173)."""
    import deep_ep
    T, H, E, K, A = 40, 128, 4, 3, 2
    x = make_tokens(T, H, seed=21)
    topk, w = make_routing(T, E, K, seed=21, masked=0.2)
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    buf = deep_ep.EPBuffer(deep_ep.LocalGroup(), num_max_tokens_per_rank=T, hidden=H, num_topk=K, explicitly_destroy=True)
    _, _, rw, handle, _ = buf.dispatch(x.to(DEV), topk_idx=topk.to(DEV), topk_weights=w.to(DEV), num_experts=E,
                                       expert_alignment=A, do_expand=True, do_zero_padding=True)
    g = torch.Generator().manual_seed(2)
    y = torch.randn((lay['num_expanded_tokens'], H), generator=g).to(torch.bfloat16)
    r = torch.rand(y.shape, generator=g)
    y[r < 0.02] = float('inf')
    y[(r >= 0.02) & (r < 0.04)] = float('-inf')
    y[(r >= 0.04) & (r < 0.05)] = float('nan')
    y[(r >= 0.05) & (r < 0.06)] = 3.3e38                     # sums overflow to inf
    bias = torch.randn((T, H), generator=g).to(torch.bfloat16)
    for b in (None, bias):
        cx, _, _ = buf.combine(y.to(DEV), handle, topk_weights=rw, bias=None if b is None else b.to(DEV))
        torch.cuda.synchronize()
        ox, _ = O.combine_fast(y, None, lay['recv_src_metadata'], T, K, b)
        got, want = bf16_bits(cx), bf16_bits(ox)
        both_nan = ((got & 0x7fff) > 0x7f80) & ((want & 0x7fff) > 0x7f80)      # any NaN equals any NaN
        assert ((got == want) | both_nan).all()
        assert both_nan.any() and ((want & 0x7fff) == 0x7f80).any()
    buf.destroy()
