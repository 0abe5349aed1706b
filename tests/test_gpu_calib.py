"""The calibration library's formulations of the fused copy kernel (destination-ordered, steered, two-pass)
must compute what the product computes: their timings are quoted as evidence, so their outputs are compared
byte for byte with the product's dispatch of the same inputs."""
import numpy as np
import pytest
import torch

from helpers import make_routing, make_tokens

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('T,H,E,K,A,masked', [(1024, 1024, 32, 4, 16, 0.0), (1000, 1536, 64, 6, 128, 0.2)])
def test_calibration_variants_reproduce_the_product_output(T, H, E, K, A, masked):
    import deep_ep
    import ep_calib
    ep_calib.init()
    dev = torch.device('cuda', 0)
    x = make_tokens(T, H, seed=5, outliers=True).to(dev)
    topk, w = make_routing(T, E, K, seed=5, masked=masked)
    topk, w = topk.to(dev), w.to(dev)
    buf = deep_ep.EPBuffer(deep_ep.LocalGroup(), num_max_tokens_per_rank=T, hidden=H, num_topk=K, use_fp8_dispatch=True,
                           explicitly_destroy=True)
    (rx, rsf), _, rw, handle, _ = buf.dispatch(x, topk_idx=topk, topk_weights=w, num_experts=E, expert_alignment=A,
                                               do_expand=True, do_zero_padding=True, fused_fp8_quant=True)
    torch.cuda.synchronize()
    want = (rx.view(torch.uint8).cpu().numpy(), rsf.cpu().numpy().view(np.uint32), rw.cpu().numpy().view(np.uint32))
    meta = handle.recv_src_metadata
    num_recv = handle.psum_num_recv_tokens_per_rank[-1:]

    def fresh():
        return (torch.full_like(rx.view(torch.uint8), 0xA5), torch.full_like(rsf, 7.0), torch.full_like(rw, 7.0))

    def args_for(ox, osf, ow):
        a = ep_calib.ScatterArgs()
        a.x, a.topk_weights = x.data_ptr(), w.data_ptr()
        a.recv_src_metadata, a.num_recv = meta.data_ptr(), num_recv.data_ptr()
        a.psum_expert = handle.psum_num_recv_tokens_per_expert.data_ptr()
        a.recv_x, a.recv_sf, a.recv_topk_weights = ox.data_ptr(), osf.data_ptr(), ow.data_ptr()
        a.num_tokens, a.hidden, a.num_topk, a.num_experts, a.expert_alignment = T, H, K, E, A
        a.num_recv_rows, a.num_out_rows, a.do_zero_padding = meta.size(0), rx.size(0), 1
        return a

    def check(name, outs):
        torch.cuda.synchronize()
        got = (outs[0].cpu().numpy(), outs[1].cpu().numpy().view(np.uint32), outs[2].cpu().numpy().view(np.uint32))
        for g, e, what in zip(got, want, ('payload', 'scales', 'weights')):
            assert np.array_equal(g, e), f'{name}: {what} differ from the product dispatch'

    outs = fresh()
    ep_calib.scatter('token_major', args_for(*outs))
    check('token_major', outs)

    q_rows = torch.empty((T, H), dtype=torch.uint8, device=dev)
    q_sf = torch.empty((T, H // 128), dtype=torch.float32, device=dev)
    for C in (128, 512, T + 24):
        flat, _, _ = ep_calib.build_order(meta, K, C, steered=False)
        steered, per_list, num_lists = ep_calib.build_order(meta, K, C, steered=True)
        for variant, order, pl, nl in (('ordered_flat', flat, 0, 0), ('ordered_steered', steered, per_list, num_lists),
                                       ('copy_ordered_flat', flat, 0, 0), ('copy_ordered_steered', steered, per_list, num_lists)):
            outs = fresh()
            a = args_for(*outs)
            a.order, a.num_entries, a.entries_per_list, a.num_lists = order.data_ptr(), order.size(0), pl, nl
            a.q_rows, a.q_sf = q_rows.data_ptr(), q_sf.data_ptr()
            if variant.startswith('copy_'):
                ep_calib.scatter('quant_rows', a)
            ep_calib.scatter(variant, a)
            check(f'{variant} chunk {C}', outs)
    # the partial variants only have to run: they write arbitrary payload or nothing
    outs = fresh()
    a = args_for(*outs)
    flat, _, _ = ep_calib.build_order(meta, K, 256, steered=False)
    steered, per_list, num_lists = ep_calib.build_order(meta, K, 256, steered=True)
    for variant, order, pl, nl in (('stores_only', flat, 0, 0), ('read_rows', flat, 0, 0), ('ordered_flat_stores_only', flat, 0, 0),
                                   ('ordered_steered_stores_only', steered, per_list, num_lists),
                                   ('ordered_steered_loads_only', steered, per_list, num_lists)):
        a.order, a.num_entries, a.entries_per_list, a.num_lists = order.data_ptr(), order.size(0), pl, nl
        ep_calib.scatter(variant, a)
    torch.cuda.synchronize()
    buf.destroy()


@pytest.mark.parametrize('T,H,E,A,masked', [(1024, 2048, 32, 16, 0.0), (700, 7168, 64, 128, 0.2)])
def test_calibration_combine_reproduces_the_product_output(T, H, E, A, masked):
    """The combine kernel body as the calibration code object builds it (top-6) gives the product's bytes; its
    loads-only form writes nothing; its stores-only form writes every row the product writes."""
    import deep_ep
    import ep_calib
    ep_calib.init()
    K = 6
    dev = torch.device('cuda', 0)
    x = make_tokens(T, H, seed=9).to(dev)
    topk, w = make_routing(T, E, K, seed=9, masked=masked)
    topk, w = topk.to(dev), w.to(dev)
    buf = deep_ep.EPBuffer(deep_ep.LocalGroup(), num_max_tokens_per_rank=T, hidden=H, num_topk=K, explicitly_destroy=True)
    rx, _, rw, handle, _ = buf.dispatch(x, topk_idx=topk, topk_weights=w, num_experts=E, expert_alignment=A,
                                        do_expand=True, do_zero_padding=True)
    y = (rx.float() * 0.5 + 0.25).to(torch.bfloat16)
    want_x, want_w, _ = buf.combine(y, handle, topk_weights=rw)
    torch.cuda.synchronize()
    num_recv = handle.psum_num_recv_tokens_per_rank[-1:]

    def args_for(ox, ow):
        a = ep_calib.CombineArgs()
        a.y, a.expanded_weights = y.data_ptr(), rw.data_ptr()
        a.recv_src_metadata, a.num_recv, a.topk_idx = handle.recv_src_metadata.data_ptr(), num_recv.data_ptr(), topk.data_ptr()
        a.combined_x, a.combined_topk_weights = ox.data_ptr(), ow.data_ptr()
        a.num_tokens, a.hidden, a.num_topk, a.num_experts = T, H, K, E
        a.num_recv_rows, a.num_in_rows, a.blocks_per_cu = handle.recv_src_metadata.size(0), y.size(0), 3
        return a

    ox, ow = torch.full_like(want_x, 7.0), torch.full_like(want_w, 7.0)
    ep_calib.combine('combine', args_for(ox, ow))
    torch.cuda.synchronize()
    assert torch.equal(ox.view(torch.int16), want_x.view(torch.int16)) and torch.equal(ow.view(torch.int32), want_w.view(torch.int32))
    # loads only: the rows of routed tokens stay as they were (tokens without any expert are zeroed by the workgroups
    # that look after them in every form)
    routed = (topk >= 0).any(dim=1)
    ox.fill_(7.0)
    ep_calib.combine('combine_loads_only', args_for(ox, ow))
    torch.cuda.synchronize()
    assert bool((ox[routed] == 7.0).all())
    # stores only: every routed token's row is written
    ox.fill_(7.0)
    ep_calib.combine('combine_stores_only', args_for(ox, ow))
    torch.cuda.synchronize()
    assert not bool((ox[routed] == 7.0).all(dim=1).any())
    with pytest.raises(ep_calib.CalibError, match='Assertion exception'):
        a = args_for(ox, ow)
        a.num_topk = 4
        ep_calib.combine('combine', a)
    buf.destroy()


def test_calibration_fills_write_every_byte():
    import ep_calib
    ep_calib.init()
    dev = torch.device('cuda', 0)
    area = torch.zeros(1 << 22, dtype=torch.uint8, device=dev)
    ep_calib.fill(area, value=0x01010101)
    assert int(area.sum()) == area.numel()
    area.zero_()
    ep_calib.fill(area, shuffled=4, value=0x02020202)
    assert int(area.sum()) == 2 * area.numel()
    for modulus, shift in ((8, 0), (32, 5)):
        area.zero_()
        ep_calib.fill_affine(area, modulus, shift, value=0x03030303)
        assert int(area.sum()) == 3 * area.numel()
    area.zero_()
    ep_calib.fronts(area, 8, 16, 7168, 16 * 7168 + 4096)
    torch.cuda.synchronize()
    rows = area[:8 * (16 * 7168 + 4096)].view(8, -1)[:, :16 * 7168]
    assert int((rows.view(torch.int32).view(8, 16, -1)[:, :, 0] == 1).sum()) == 8 * 16       # first word of every row
    src = torch.zeros(4096 * 3, dtype=torch.uint8, device=dev)
    dst = torch.full((4096 * 7,), 9, dtype=torch.uint8, device=dev)
    ep_calib.mixed(src, dst, 2, 7)
    assert int(dst.sum()) == 0
    with pytest.raises(ep_calib.CalibError, match='Assertion exception'):
        ep_calib.fill(area[:1000])
