"""Headline benchmark: EP dispatch (fused BF16->FP8 e4m3) + BF16 combine of one GPU's share at
16384 tokens x hidden 7168, top-6 of 256 experts, expert alignment 128.

  python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one dispatch followed by one combine over synthetic inputs that are already resident in
HBM.  After W warm-up steps exactly K steps are timed between two device synchronisations; the
JSON line printed at the end carries the whole-step throughput (`value`, algorithmic bytes of both
phases over the wall time of a step), the roofline of the dominant kernel measured with HIP events
on the stream the kernels run on, the same for every kernel, and the CPU oracle timed on this
machine's host cores on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, 'deepep-ascend_amd'), os.path.join(ROOT, 'tests')):
    if p not in sys.path:
        sys.path.insert(0, p)

import numpy as np  # noqa: E402
import torch  # noqa: E402

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch come from the committed rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary of a workload
# (lines "traffic_bytes <kernel> <bytes>"), and only while that summary was taken from the kernel sources
# that are being run (line "kernel_source_sha256 <hash>"); otherwise the field is null.
TRAFFIC_PROFILES = {'c3_headline': 'headline_dispatch_combine_hbm_traffic.txt',
                    'c3_prequantised': 'headline_prequantised_counters.txt',
                    'c2_bf16_top8': 'c2_bf16_top8_counters.txt',
                    'c4_decode_zipf': 'c4_decode_zipf_counters.txt',
                    'c5_ep32_share': 'ep32_share_counters.txt',
                    'c5_ep32_node': 'ep32_node_counters.txt'}
KERNEL_SOURCES = ('deepep-ascend_amd/csrc/ep_kernels.hip', 'deepep-ascend_amd/csrc/ep_args.h',
                  'deepep-ascend_amd/csrc/ep_fp8.h')


def kernel_source_sha256():
    import hashlib
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), 'rb') as f:
            h.update(f.read())
    return h.hexdigest()


def measured_traffic(workload):
    """{kernel: HBM bytes per launch} from the committed counter summary of this workload, or {} when there
    is none or it was taken from other kernel sources."""
    name = TRAFFIC_PROFILES.get(workload)
    path = os.path.join(ROOT, 'profiles', name) if name else None
    if not path or not os.path.exists(path):
        return {}, 'no counter summary committed for this workload'
    sha, out = None, {}
    with open(path) as f:
        for line in f:
            w = line.split()
            if len(w) == 2 and w[0] == 'kernel_source_sha256':
                sha = w[1]
            elif len(w) == 3 and w[0] == 'traffic_bytes':
                out[w[1]] = float(w[2])
    if sha != kernel_source_sha256():
        return {}, f'profiles/{name} was taken from other kernel sources'
    return out, f'profiles/{name}'
WORKLOADS = {
    # name: (T, H, E, K, A, fp8)
    'c3_headline': (16384, 7168, 256, 6, 128, True),
    'c3_prequantised': (16384, 7168, 256, 6, 128, True),   # the caller quantises: dispatch of (FP8 rows, scale packs)
    'c2_bf16_top8': (4096, 7168, 256, 8, 128, False),
    'c1_small': (128, 256, 8, 2, 1, False),
    'c4_decode_zipf': (128, 7168, 256, 8, 128, True),
    'c5_ep32_share': (16384, 7168, 256, 6, 128, True),     # 32 partitions of 8 experts, this GPU = partition 5
    'c5_ep32_node': (16384, 7168, 256, 6, 128, True),      # all 32 partitions on this GPU, connected
}


def dispatch_bytes(T, H, K, n_valid, n_recv, fp8, fused):
    s_in = 2 if (fused or not fp8) else 1
    s_out = 1 if fp8 else 2
    sfb = (H // 128) * 4 if fp8 else 0
    b = T * H * s_in + T * K * (8 + 4) + n_valid * (H * s_out + sfb + 4) + n_recv * (K + 2) * 4 + 2 * T * K * 4
    if fp8 and not fused:
        b += T * sfb
    return b


def combine_bytes(T, H, K, n_valid, n_recv, n_bias, weights):
    b = n_valid * H * 2 + T * H * 2 * (1 + n_bias) + n_recv * (K + 2) * 4 + T * K * 8
    if weights:
        b += n_valid * 4 + T * K * 4
    return b


def make_inputs(T, H, E, K, seed=0):
    from helpers import make_routing, make_tokens
    x = make_tokens(T, H, seed=seed, outliers=True)
    topk, w = make_routing(T, E, K, seed=seed)
    return x, topk, w


def cpu_small_case():
    """The reference's CPU-runnable case (128 tokens x 256, 8 experts, top-2, alignment 1, BF16 dispatch then
    combine of the dispatched rows) on the host cores: median of 20 passes of the oracle after 3 untimed ones."""
    from oracle import ep_oracle as O
    T, H, E, K, A, _ = WORKLOADS['c1_small']
    x, topk, w = make_inputs(T, H, E, K, seed=1)
    ts = []
    for k in range(3 + 20):             # three untimed passes, then the median of twenty
        t0 = time.perf_counter()
        lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
        rx, _, rw = O.rank_share_dispatch(x.view(torch.int16).numpy(), None, w.numpy(), lay)
        O.combine_fast(torch.from_numpy(rx).view(torch.bfloat16), torch.from_numpy(rw), lay['recv_src_metadata'], T, K)
        if k >= 3:
            ts.append(time.perf_counter() - t0)
    n_valid = int(lay['num_unaligned_recv_tokens_per_expert'].sum())
    nbytes = dispatch_bytes(T, H, K, n_valid, lay['num_recv_tokens'], False, False) + \
        combine_bytes(T, H, K, n_valid, lay['num_recv_tokens'], 0, True)
    med = sorted(ts)[len(ts) // 2]
    return {'workload': 'c1_small', 'ms': round(med * 1e3, 3), 'gbs': round(nbytes / med / 1e9, 3)}


def cpu_model():
    try:
        with open('/proc/cpuinfo') as f:
            for line in f:
                if line.startswith('model name'):
                    return line.split(':', 1)[1].strip()
    except OSError:
        pass
    return 'unknown'


def cpu_baseline(H, E, K, A, fp8, sample_tokens, passes=5):
    """The oracle on the host cores over `sample_tokens` tokens of the same workload: one untimed pass, then the
    median of `passes` timed ones (dispatch + combine); and the reference's own CPU-runnable case."""
    from oracle import ep_oracle as O
    torch.set_num_threads(os.cpu_count())
    x, topk, w = make_inputs(sample_tokens, H, E, K, seed=1)
    g = torch.Generator().manual_seed(2)
    y = None
    times = []
    for k in range(1 + passes):
        t0 = time.perf_counter()
        lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, sample_tokens)
        if fp8:
            q, s = O.quantise(x)
            rx, rs, rw = O.rank_share_dispatch(q.numpy(), s.numpy().view(np.uint32), w.numpy(), lay)
        else:
            rx, rs, rw = O.rank_share_dispatch(x.view(torch.int16).numpy(), None, w.numpy(), lay)
        t1 = time.perf_counter()
        if y is None:
            y = torch.randn((lay['num_expanded_tokens'], H), generator=g).to(torch.bfloat16)
        t2 = time.perf_counter()
        O.combine_fast(y, torch.from_numpy(rw), lay['recv_src_metadata'], sample_tokens, K)
        t3 = time.perf_counter()
        if k >= 1:
            times.append((t1 - t0 + t3 - t2, t1 - t0, t3 - t2))
    times.sort()
    med, med_d, med_c = times[len(times) // 2]
    n_valid = int(lay['num_unaligned_recv_tokens_per_expert'].sum())
    n_recv = lay['num_recv_tokens']
    nbytes = dispatch_bytes(sample_tokens, H, K, n_valid, n_recv, fp8, True) + combine_bytes(sample_tokens, H, K, n_valid, n_recv, 0, True)
    return {'value': round(nbytes / med / 1e9, 3), 'unit': 'GB/s', 'cores': torch.get_num_threads(), 'kind': 'port',
            'cpu_model': cpu_model(), 'passes': passes, 'median_s': round(med, 3),
            'sample': f'1 untimed pass, then the median of {passes} passes over {sample_tokens} tokens of the workload: '
                      f'dispatch {med_d:.2f} s + combine {med_c:.2f} s of numpy/torch-CPU oracle '
                      f'(os.cpu_count()={os.cpu_count()})',
            'small_case': cpu_small_case()}


def calib_scatter_args(ep_calib, xg, wg, handle, recv_x, recv_sf, recv_w, T, H, K, E, A):
    """The fused dispatch of this run as the calibration library's kernels take it (plain pointers; the tensors
    are returned as well so that they outlive the launches)."""
    a = ep_calib.ScatterArgs()
    num_recv = handle.psum_num_recv_tokens_per_rank[-1:]
    keep = (xg, wg, handle.recv_src_metadata, num_recv, handle.psum_num_recv_tokens_per_expert, recv_x, recv_sf, recv_w)
    a.x, a.topk_weights = xg.data_ptr(), wg.data_ptr()
    a.recv_src_metadata, a.num_recv = handle.recv_src_metadata.data_ptr(), num_recv.data_ptr()
    a.psum_expert = handle.psum_num_recv_tokens_per_expert.data_ptr()
    a.recv_x, a.recv_sf, a.recv_topk_weights = recv_x.data_ptr(), recv_sf.data_ptr(), recv_w.data_ptr()
    a.num_tokens, a.hidden, a.num_topk, a.num_experts, a.expert_alignment = T, H, K, E, A
    a.num_recv_rows, a.num_out_rows, a.do_zero_padding = handle.recv_src_metadata.size(0), recv_x.size(0), 1
    return a, keep


def dispatch_ceiling(ep_calib, timed, n, cargs, us_scatter):
    """What bounds the token-major copy kernel, from two kernels of the calibration code object run here: its
    store stream alone (the same tasks storing to the same slots, nothing read but the slots) and its loads
    of x alone.  On this memory system reads and writes share the time: the sum is the kernel's floor."""
    med = lambda v: v[len(v) // 2]  # noqa: E731
    st = med(timed(lambda: ep_calib.scatter('stores_only', cargs), n))
    rd = med(timed(lambda: ep_calib.scatter('read_rows', cargs), n))
    return {'stores_only_us': round(st, 2), 'read_us': round(rd, 2), 'sum_us': round(st + rd, 2),
            'copy_kernel_us': round(us_scatter, 2), 'copy_kernel_over_sum': round(us_scatter / (st + rd), 3),
            'kernels': 'ep_calib_scatter_stores_only, ep_calib_read_rows (ep_calib.hsaco), isolated flushed medians'}


def calib_combine_args(ep_calib, y, recv_w, handle, combined_x, combined_w, T, H, K, E, blocks_per_cu):
    """The combine of this run as the calibration library's kernels take it."""
    a = ep_calib.CombineArgs()
    num_recv = handle.psum_num_recv_tokens_per_rank[-1:]
    keep = (y, recv_w, handle.recv_src_metadata, num_recv, handle.topk_idx, combined_x, combined_w)
    a.y, a.expanded_weights = y.data_ptr(), recv_w.data_ptr()
    a.recv_src_metadata, a.num_recv, a.topk_idx = handle.recv_src_metadata.data_ptr(), num_recv.data_ptr(), handle.topk_idx.data_ptr()
    a.combined_x, a.combined_topk_weights = combined_x.data_ptr(), combined_w.data_ptr()
    a.num_tokens, a.hidden, a.num_topk, a.num_experts = T, H, K, E
    a.num_recv_rows, a.num_in_rows, a.blocks_per_cu = handle.recv_src_metadata.size(0), y.size(0), blocks_per_cu
    return a, keep


def combine_ceiling(ep_calib, timed, n, cargs, us_combine):
    """The combine kernel taken apart the same way: its row fetches (with the sums) alone and its stores alone, from
    two kernels of the calibration code object that run the product's kernel body.  The fetches run as the product is
    launched (workgroups a CU capped); the stores alone are timed uncapped: capped, that launch waits on its slot
    lookups (about 100 us) and says nothing about the store stream."""
    med = lambda v: v[len(v) // 2]  # noqa: E731
    ld = med(timed(lambda: ep_calib.combine('combine_loads_only', cargs), n))
    cap = cargs.blocks_per_cu
    cargs.blocks_per_cu = 0
    st = med(timed(lambda: ep_calib.combine('combine_stores_only', cargs), n))
    cargs.blocks_per_cu = cap
    return {'loads_only_us': round(ld, 2), 'stores_only_us': round(st, 2), 'sum_us': round(ld + st, 2),
            'combine_kernel_us': round(us_combine, 2), 'combine_kernel_over_sum': round(us_combine / (ld + st), 3),
            'kernels': f'ep_calib_combine_k6_loads_only ({cap} workgroups a CU, as the library launches its own), '
                       'ep_calib_combine_k6_stores_only (uncapped) (ep_calib.hsaco), isolated flushed medians'}


def calibrate_write(ep_calib, timed, n, cargs, T, H, K, n_valid, n_recv, pad_bytes, dev, us_scatter, meta):
    """Pure writes of the byte count the fused FP8 copy kernel writes (payload, scales, weights, zero padding),
    same sampling as the kernels: 4 KiB chunks in address order, in scrambled order, 256 write fronts in lock
    step, a mixed read/write stream in address order, torch's fill; then the formulations of the copy kernel
    that write in destination order (one pass, and quantise-then-copy), whole and taken apart."""
    wbytes = n_valid * (H + (H // 128) * 4 + 4) + pad_bytes
    seq_bytes = -(-wbytes // 4096) * 4096
    pow2_bytes = 4096 << (seq_bytes // 4096 - 1).bit_length()          # the scrambled order needs 2^k chunks
    area = torch.empty(pow2_bytes, dtype=torch.uint8, device=dev)
    med = lambda v: v[len(v) // 2]  # noqa: E731
    res = {'copy_kernel_write_bytes': wbytes}

    def entry(name, us, nbytes, note):
        res[name] = {'us': round(us, 2), 'bytes': nbytes, 'gbs': round(nbytes / us / 1e3, 1), 'what': note}

    entry('ep_calib_fill', med(timed(lambda: ep_calib.fill(area[:seq_bytes]), n)), seq_bytes,
          '4 KiB per workgroup, one 16-byte non-temporal store per thread, address order')
    entry('ep_calib_fill_shuffled', med(timed(lambda: ep_calib.fill(area, shuffled=1), n)), pow2_bytes,
          'the same chunks in a scrambled order')
    for unit in (4, 16, 256):                                         # 16 KiB, 64 KiB, 1 MiB
        entry(f'ep_calib_fill_shuffled_{unit * 4}KiB', med(timed(lambda: ep_calib.fill(area, shuffled=unit), n)),
              pow2_bytes, f'runs of {unit} chunks ({unit * 4} KiB) kept together, the runs scrambled')
    for modulus in (8, 32):
        entry(f'ep_calib_fill_affine_mod{modulus}', med(timed(lambda: ep_calib.fill_affine(area, modulus), n)), pow2_bytes,
              f'scrambled 4 KiB chunks again, but any {modulus} consecutive workgroups write chunks with {modulus} different '
              f'indices modulo {modulus}' + (' (every XCD keeps the chunks address order gives it)' if modulus == 8 else
                                            ' (concurrent writes spread evenly over 32 consecutive 4 KiB blocks: the interleave of the memory)'))
    for nf in (8, 64):
        frows = pow2_bytes // 4096 // nf
        entry(f'ep_calib_fronts_{nf}x4KiB', med(timed(lambda: ep_calib.fronts(area, nf, frows, 4096, frows * 4096), n)), nf * frows * 4096,
              f'{nf} regions filling up in lock step, a 4 KiB row per workgroup')
    rows = min(448, area.numel() // (256 * H))
    entry('ep_calib_fronts_256', med(timed(lambda: ep_calib.fronts(area, 256, rows, H, rows * H), n)), 256 * rows * H,
          f'256 regions filling up in lock step, one {H}-byte row per workgroup (what a gather-formulated dispatch writes)')
    src = torch.zeros(-(-seq_bytes * 2 // 7 // 4096) * 4096 + 4096, dtype=torch.uint8, device=dev)
    us = med(timed(lambda: ep_calib.mixed(src, area[:seq_bytes], 2, 7), n))
    res['ep_calib_mixed_2r7w'] = {'us': round(us, 2), 'bytes_written': seq_bytes, 'bytes_read': seq_bytes * 2 // 7,
                                  'gbs': round(seq_bytes * 9 / 7 / us / 1e3, 1),
                                  'what': 'address-ordered 4 KiB chunks, 2 read per 7 written (the copy kernel\'s ratio): '
                                          'the friendliest stream with the kernel\'s traffic'}
    entry('torch_fill', med(timed(lambda: area[:seq_bytes].zero_(), n)), seq_bytes, 'torch zero_() of the same bytes')
    del src, area

    def variant(name, what, prep=None):
        us = med(timed(lambda: ep_calib.scatter(name, cargs), n))
        res['ep_calib_' + name if not prep else prep] = {'us': round(us, 2), 'what': what}

    variant('token_major', 'the product copy kernel body built into the calibration code object (cached-replay form)')
    variant('stores_only', 'the copy kernel without its loads of x: same tasks, same stores')
    variant('read_rows', 'the copy kernel\'s loads of x alone')
    res['ep_scatter_quant'] = {'us': round(us_scatter, 2), 'what': 'the copy kernel (reads x, writes the same bytes)'}
    # destination order: tasks sorted by slot inside chunks of tokens (a chunk of C tokens leaves one run of about
    # C * K / E rows in every expert's region)
    q_rows = torch.empty((T, H), dtype=torch.uint8, device=dev)
    q_sf = torch.empty((T, H // 128), dtype=torch.float32, device=dev)
    cargs.q_rows, cargs.q_sf = q_rows.data_ptr(), q_sf.data_ptr()
    variant('quant_rows', 'two passes, pass 1: every row quantised once, token order, into staging rows')
    for C in (512, 2048, T):
        flat, _, _ = ep_calib.build_order(meta, K, C, steered=False)
        cargs.order, cargs.num_entries, cargs.entries_per_list, cargs.num_lists = flat.data_ptr(), flat.size(0), 0, 0
        tag = f'chunk{C}'
        variant('ordered_flat', f'one task per destination row, destination order inside chunks of {C} tokens',
                f'ep_calib_ordered_flat_{tag}')
        variant('ordered_flat_stores_only', 'the same without the loads of x', f'ep_calib_ordered_flat_stores_only_{tag}')
        variant('copy_ordered_flat', 'two passes, pass 2: staged FP8 rows copied in that order', f'ep_calib_copy_ordered_flat_{tag}')
        if C < T:
            st, per_list, num_lists = ep_calib.build_order(meta, K, C, steered=True)
            cargs.order, cargs.num_entries = st.data_ptr(), st.size(0)
            cargs.entries_per_list, cargs.num_lists = per_list, num_lists
            variant('ordered_steered', 'the same with all readers of a token on one XCD (x is fetched from memory once)',
                    f'ep_calib_ordered_steered_{tag}')
            variant('ordered_steered_stores_only', 'without the loads', f'ep_calib_ordered_steered_stores_only_{tag}')
            variant('ordered_steered_loads_only', 'without the stores (no zero padding either)',
                    f'ep_calib_ordered_steered_loads_only_{tag}')
            variant('copy_ordered_steered', 'two passes, pass 2, steered', f'ep_calib_copy_ordered_steered_{tag}')
            del st
        del flat
    return res


def timed_us(fn, n):
    """Average duration of fn in microseconds, from events on the current stream (the launch stream)."""
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    v = [a.elapsed_time(b) * 1e3 for a, b in evs]
    return sum(v) / len(v)


def bench_partitioned(args, T, H, E, K, A, R=32, rank=5):
    """One GPU's share of EP-R: pack into R partition-major regions + expand the own region, then the
    owner-side partial reduce + the token-side final reduce over a combine buffer whose other partials are
    synthetic.  Not the headline line: printed for the record when asked for."""
    import deep_ep
    dev = torch.device('cuda', 0)
    x, topk, w = make_inputs(T, H, E, K)
    xg, tg, wg = x.to(dev), topk.to(dev), w.to(dev)
    buf = deep_ep.EPBuffer(deep_ep.LocalGroup(rank, R), num_max_tokens_per_rank=T, hidden=H, num_topk=K,
                           use_fp8_dispatch=True, explicitly_destroy=True)
    kw = dict(num_experts=E, num_max_tokens_per_rank=T, expert_alignment=A, do_expand=True, do_zero_padding=True,
              fused_fp8_quant=True)
    (rx, rsf), _, rw, handle, _ = buf.dispatch(xg, topk_idx=tg, topk_weights=wg, **kw)
    y = torch.randn((rx.size(0), H), device=dev).to(torch.bfloat16)
    arena = buf.runtime.buffer_tensor()
    ctok = H * 2 + -(-4 * K // 32) * 32
    arena[:min(K, R) * T * ctok].view(torch.int16).random_(0, 0x3f80)       # finite BF16 partials everywhere
    torch.cuda.synchronize()
    n_send = int((handle.dst_buffer_slot_idx >= 0).sum())
    n_recv = int(handle.psum_num_recv_tokens_per_rank[-1])
    n_valid = int(handle.num_unaligned_recv_tokens_per_expert.sum())
    tok = H + 224 + 96
    b_pack = T * H * 2 + T * K * 12 + n_send * tok
    b_expand = n_recv * tok + n_valid * (H + 224 + 4) + n_recv * (K + 2) * 4
    b_partial = n_valid * H * 2 + n_recv * ctok + n_recv * (K + 2) * 4
    b_final = n_send * ctok + T * H * 2 + T * K * 8 + T * K * 4

    def step():
        _, _, rw2, h, _ = buf.dispatch(xg, topk_idx=tg, topk_weights=wg, **kw)
        buf.combine(y, h, topk_weights=rw2)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    us_d = timed_us(lambda: buf.dispatch(xg, topk_idx=tg, topk_weights=wg, **kw), args.steps)
    us_c = timed_us(lambda: buf.combine(y, handle, topk_weights=rw), args.steps)
    # the send side alone (layout + the pack kernel, the largest of this workload): a deferred dispatch enqueues
    # exactly that; its epilogue runs outside the bracket
    pend = []

    def send_side():
        pend.append(buf.dispatch(xg, topk_idx=tg, topk_weights=wg, async_with_compute_stream=True, defer_epilogue=True, **kw))

    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for a, b in evs:
        a.record()
        send_side()
        b.record()
        pend.pop().current_stream_wait()
    torch.cuda.synchronize()
    us_send = sorted(a.elapsed_time(b) * 1e3 for a, b in evs)[len(evs) // 2]
    traffic, traffic_source = measured_traffic(args.workload)
    roofline = {'kernel': 'ep_scatter_quant_pack', 'bound': 'hbm', 'achieved': round(b_pack / us_send / 1e3, 1),
                'peak': HBM_PEAK_GBS, 'unit': 'GB/s', 'frac': round(b_pack / us_send / 1e3 / HBM_PEAK_GBS, 4),
                'traffic': traffic.get('ep_scatter_quant_pack'), 'traffic_source': traffic_source, 'us': round(us_send, 2),
                'measured': 'events around the send side of a dispatch (layout kernels + pack kernel), median'}
    out = {'metric': 'dispatch & combine GB/s, one GPU share of EP32 (pack 32 regions + expand own; partial + final reduce)',
           'value': round((b_pack + b_expand + b_partial + b_final) / ms / 1e6, 1), 'unit': 'GB/s', 'n_gpus': 1,
           'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': round(ms, 4), 'higher_is_better': True,
           'scaling': 'weak', 'vs_baseline': None, 'dtype': 'fp8_e4m3+bf16 payload, fp32 accumulate', 'data': 'synthetic',
           'config': {'workload': args.workload, 'tokens': T, 'hidden': H, 'experts': E, 'topk': K,
                      'expert_alignment': A, 'partitions': R, 'partition_idx': rank, 'packed_rows': n_send,
                      'received_rows': n_recv, 'valid_expanded_rows': n_valid},
           'roofline': roofline,
           'phases': {'dispatch_us': round(us_d, 2), 'dispatch_bytes': b_pack + b_expand,
                      'dispatch_gbs': round((b_pack + b_expand) / us_d / 1e3, 1),
                      'combine_us': round(us_c, 2), 'combine_bytes': b_partial + b_final,
                      'combine_gbs': round((b_partial + b_final) / us_c / 1e3, 1)}}
    buf.destroy()
    print(json.dumps(out))


def bench_node(args, T, H, E, K, A, R=32, rank=5):
    """All R partitions of the EP group on this GPU, connected: every partition dispatches T tokens, so each
    receives its real share (about T*K rows from R sources) and reduces it.  A step runs the four phases for
    every partition in turn; the phases of one partition are timed with events.  For the record, not the
    headline line."""
    import deep_ep
    dev = torch.device('cuda', 0)
    x, topk, w = make_inputs(T, H, E, K)
    xg, tg, wg = x.to(dev), topk.to(dev), w.to(dev)
    node = deep_ep.LocalNode(R)
    bufs = [deep_ep.EPBuffer(node.group(r), num_max_tokens_per_rank=T, hidden=H, num_topk=K, use_fp8_dispatch=True,
                             explicitly_destroy=True) for r in range(R)]
    kw = dict(num_experts=E, num_max_tokens_per_rank=T, expert_alignment=A, do_expand=True, do_zero_padding=True,
              fused_fp8_quant=True, async_with_compute_stream=True, defer_epilogue=True)
    y = None
    phases = {k: [] for k in ('send', 'recv', 'partial', 'final')}

    def ev():
        return torch.cuda.Event(enable_timing=True)

    def node_step(timed):
        nonlocal y
        marks = [ev() for _ in range(8)]
        sends = []
        for r in range(R):
            if r == rank:
                marks[0].record()
            sends.append(bufs[r].dispatch(xg, topk_idx=tg, topk_weights=wg, **kw))
            if r == rank:
                marks[1].record()
        handles, weights = [], []
        for r in range(R):
            if r == rank:
                marks[2].record()
            (rx, rsf), _, rw, h = sends[r].current_stream_wait()
            if r == rank:
                marks[3].record()
            if y is None or y.size(0) < rx.size(0):
                y = torch.randn((rx.size(0) + 4096, H), device=dev).to(torch.bfloat16)
            handles.append(h)
            weights.append(rw)
            del rx, rsf
        partials = []
        for r in range(R):
            if r == rank:
                marks[4].record()
            partials.append(bufs[r].combine(y[:handles[r].num_expanded_tokens], handles[r], topk_weights=weights[r],
                                            async_with_compute_stream=True, defer_epilogue=True))
            if r == rank:
                marks[5].record()
        for r in range(R):
            if r == rank:
                marks[6].record()
            partials[r].current_stream_wait()
            if r == rank:
                marks[7].record()
        if timed:
            torch.cuda.synchronize()
            for i, k in enumerate(('send', 'recv', 'partial', 'final')):
                phases[k].append(marks[2 * i].elapsed_time(marks[2 * i + 1]) * 1e3)
        return handles[rank]

    for _ in range(args.warmup):
        handle = node_step(False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        handle = node_step(True)
    torch.cuda.synchronize()
    node_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    n_send = int((handle.dst_buffer_slot_idx >= 0).sum())
    n_recv = int(handle.psum_num_recv_tokens_per_rank[-1])
    n_valid = int(handle.num_unaligned_recv_tokens_per_expert.sum())
    tok, ctok = H + 224 + 96, H * 2 + -(-4 * K // 32) * 32
    nbytes = {'send': T * H * 2 + T * K * 12 + n_send * tok,
              'recv': n_recv * tok + n_valid * (H + 224 + 4) + 2 * n_recv * (K + 2) * 4 + n_recv * K * 8,
              'partial': n_valid * H * 2 + n_recv * ctok + n_recv * (K + 2) * 4,
              'final': n_send * ctok + T * H * 2 + T * K * 12}
    us = {k: sum(v) / len(v) for k, v in phases.items()}
    share_ms = node_ms / R
    traffic, traffic_source = measured_traffic(args.workload)
    roofline = {'kernel': f'ep_combine_partial_k{K}', 'bound': 'hbm', 'achieved': round(nbytes['partial'] / us['partial'] / 1e3, 1),
                'peak': HBM_PEAK_GBS, 'unit': 'GB/s', 'frac': round(nbytes['partial'] / us['partial'] / 1e3 / HBM_PEAK_GBS, 4),
                'traffic': traffic.get(f'ep_combine_partial_k{K}'), 'traffic_source': traffic_source, 'us': round(us['partial'], 2),
                'measured': 'events around the owner-side reduce of one partition inside the timed node steps, mean'}
    out = {'metric': 'dispatch & combine GB/s, one partition of EP32 at its real share (all 32 partitions on one GPU, '
                     'rows and partials stored straight into peer arenas)',
           'value': round(sum(nbytes.values()) / share_ms / 1e6, 1), 'unit': 'GB/s', 'n_gpus': 1, 'steps': args.steps,
           'warmup': args.warmup, 'ms_per_step': round(share_ms, 4), 'higher_is_better': True, 'scaling': 'weak',
           'vs_baseline': None, 'dtype': 'fp8_e4m3+bf16 payload, fp32 accumulate', 'data': 'synthetic',
           'config': {'workload': args.workload, 'tokens_per_partition': T, 'hidden': H, 'experts': E, 'topk': K,
                      'expert_alignment': A, 'partitions': R, 'timed_partition': rank, 'packed_rows_sent': n_send,
                      'rows_received': n_recv, 'valid_expanded_rows': n_valid, 'node_step_ms': round(node_ms, 3),
                      'ms_per_step_is': 'node step / partitions (host clock)'},
           'roofline': roofline,
           'phases': {k: {'us': round(us[k], 1), 'bytes': nbytes[k], 'gbs': round(nbytes[k] / us[k] / 1e3, 1)}
                      for k in us}}
    for b in bufs:
        b.destroy()
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=10)
    ap.add_argument('--workload', default='c3_headline', choices=sorted(WORKLOADS))
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--cpu-sample-tokens', type=int, default=16384)
    ap.add_argument('--no-cpu-sync', action='store_true', help='dispatch without the host count wait')
    ap.add_argument('--graph', action='store_true',
                    help='record the step (dispatch without host sync + combine) into a HIP graph and replay it')
    ap.add_argument('--no-flush', action='store_true',
                    help='per-kernel samples back to back, without rewriting a 1 GiB scratch buffer between them')
    ap.add_argument('--calibrate-copy', action='store_true',
                    help='also run a plain 1 GiB device copy (known traffic) to scale rocprof byte counters')
    ap.add_argument('--calibrate-write', action='store_true',
                    help='also time the kernels of the calibration library: pure writes of the copy kernel\'s byte '
                         'count in several orders, a mixed read/write stream, and the destination-ordered and '
                         'two-pass formulations of the copy kernel')
    ap.add_argument('--combine-blocks-per-cu', type=int, default=None,
                    help='tuning: workgroups of a combine kernel a CU holds at once (library default: by top-k; 0: no cap)')
    ap.add_argument('--samples', type=int, default=50, help='isolated, cache-flushed launches per kernel')
    args = ap.parse_args()
    if args.graph:
        args.no_cpu_sync = True     # a graph cannot hold the host's wait for the counts
    if args.gpus != 1 or int(os.environ.get('WORLD_SIZE', '1')) != 1:
        print('bench.py measures one GPU\'s share of the EP path; run it with --gpus 1 (no collectives exist here)',
              file=sys.stderr)
        sys.exit(2)

    import deep_ep
    if args.combine_blocks_per_cu is not None:
        deep_ep._C.set_combine_blocks_per_cu(args.combine_blocks_per_cu)
    T, H, E, K, A, fp8 = WORKLOADS[args.workload]
    dev = torch.device('cuda', 0)
    torch.cuda.set_device(dev)
    if args.calibrate_copy:
        src = torch.zeros(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)          # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
    if args.workload == 'c5_ep32_share':
        bench_partitioned(args, T, H, E, K, A)
        return
    if args.workload == 'c5_ep32_node':
        bench_node(args, T, H, E, K, A)
        return
    x, topk, w = make_inputs(T, H, E, K)
    xg, tg, wg = x.to(dev), topk.to(dev), w.to(dev)
    fused = fp8 and args.workload != 'c3_prequantised'
    if fp8 and not fused:
        # the drop-in form of the reference: the caller's quantiser, scales handed over as 2-byte packs
        xq, xs = deep_ep.utils.math.per_token_cast_to_fp8(xg)
        xg = (xq, xs.view(torch.int16))
    buf = deep_ep.EPBuffer(deep_ep.LocalGroup(), num_max_tokens_per_rank=T, hidden=H, num_topk=K,
                           use_fp8_dispatch=fp8, explicitly_destroy=True)
    kw = dict(num_experts=E, num_max_tokens_per_rank=T, expert_alignment=A, do_expand=True, do_zero_padding=True,
              fused_fp8_quant=fused)

    def dispatch(handle=None):
        if handle is None:
            return buf.dispatch(xg, topk_idx=tg, topk_weights=wg, do_cpu_sync=not args.no_cpu_sync, **kw)
        return buf.dispatch(xg, topk_weights=wg, handle=handle, do_expand=True, do_zero_padding=True,
                            fused_fp8_quant=fused)

    recv, _, recv_w, handle, _ = dispatch()
    n_exp = (recv[0] if fp8 else recv).size(0)
    y = torch.randn((n_exp, H), generator=torch.Generator(device=dev).manual_seed(1), device=dev).to(torch.bfloat16)
    torch.cuda.synchronize()
    n_valid = int(handle.num_unaligned_recv_tokens_per_expert.sum().item())
    n_recv = int(handle.psum_num_recv_tokens_per_rank[-1].item())
    n_exp_exact = int(handle.psum_num_recv_tokens_per_expert[-1].item() + A - 1) // A * A
    b_d = dispatch_bytes(T, H, K, n_valid, n_recv, fp8, fused)
    b_c = combine_bytes(T, H, K, n_valid, n_recv, 0, True)
    pad_bytes = (n_exp_exact - n_valid) * (H * (1 if fp8 else 2) + ((H // 128) * 4 if fp8 else 0) + 4)

    def step():
        r, _, rw, h, _ = dispatch()
        buf.combine(y, h, topk_weights=rw)

    # The timed region: K steps back to back.  Events on the launch stream split every step into its
    # dispatch phase (layout kernels, host count read, copy kernel) and its combine kernel.
    # (two events a step: a step ends where the next one starts; one more event closes the last step)
    marks = [tuple(torch.cuda.Event(enable_timing=True) for _ in range(2)) for _ in range(args.steps + 1)]

    def marked_step(m):
        m[0].record()
        r, _, rw, h, _ = dispatch()
        m[1].record()
        buf.combine(y, h, topk_weights=rw)

    graph = None
    if args.graph:
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            step()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
    for _ in range(args.warmup):
        graph.replay() if graph is not None else step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for m in marks[:-1]:
        graph.replay() if graph is not None else marked_step(m)
    if graph is None:
        marks[-1][0].record()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    loop_dispatch = loop_combine = None
    if graph is None:
        loop_dispatch = sorted(m[0].elapsed_time(m[1]) * 1e3 for m in marks[:-1])
        loop_combine = sorted(m[1].elapsed_time(n[0]) * 1e3 for m, n in zip(marks[:-1], marks[1:]))

    # Isolated samples: each kernel alone (the copy kernel as the epilogue of a deferred dispatch, and again as
    # what a cached dispatch enqueues).  Ten untimed launches, then --samples timed ones; before each a 1 GiB scratch buffer is rewritten, so no sample finds its inputs in
    # the L2 or the memory-side cache (the reference's benchmark does the same: tests/ep/test_ep.py:79-80,
    # 415-421).  The median is reported (the mean beside it).
    scratch = None if args.no_flush else torch.empty(1 << 30, dtype=torch.uint8, device=dev)

    def timed(fn, n, warm=10):
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
        for _ in range(warm):
            fn()
        for a, b in evs:
            if scratch is not None:
                scratch.zero_()
            a.record()
            fn()
            b.record()
        torch.cuda.synchronize()
        return sorted(a.elapsed_time(b) * 1e3 for a, b in evs)      # microseconds

    def timed_copy_kernel(n, warm=10):
        # The copy kernel of a non-cached dispatch by itself: the layout kernels of a deferred dispatch run in
        # front of the bracket, its epilogue (the copy kernel, then the host's read of the counts) inside.
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
        for k in range(warm + n):
            if scratch is not None:
                scratch.zero_()
            ev = buf.dispatch(xg, topk_idx=tg, topk_weights=wg, do_cpu_sync=not args.no_cpu_sync,
                              async_with_compute_stream=True, defer_epilogue=True, **kw)
            if k >= warm:
                evs[k - warm][0].record()
            ev.current_stream_wait()
            if k >= warm:
                evs[k - warm][1].record()
        torch.cuda.synchronize()
        return sorted(a.elapsed_time(b) * 1e3 for a, b in evs)

    n_k = args.samples
    t_scatter = timed_copy_kernel(n_k)
    t_scatter_cached = timed(lambda: dispatch(handle), n_k)
    t_combine = timed(lambda: buf.combine(y, handle, topk_weights=recv_w), n_k)
    t_dispatch_full = timed(lambda: dispatch(), n_k)
    # the layout kernels alone: a deferred dispatch enqueues them and returns; its copy epilogue runs outside the
    # timed bracket (a one-element list carries the pending event from the timed call to the clean-up)
    pending = []

    def layout_only():
        if pending:
            pending.pop().current_stream_wait()
        pending.append(buf.dispatch(xg, topk_idx=tg, topk_weights=wg, do_cpu_sync=not args.no_cpu_sync,
                                    async_with_compute_stream=True, defer_epilogue=True, **kw))

    def timed_layout(n, warm=10):
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
        for k in range(warm + n):
            if pending:
                pending.pop().current_stream_wait()                   # the previous launch's epilogue, untimed
            if scratch is not None:
                scratch.zero_()
            if k >= warm:
                evs[k - warm][0].record()
            layout_only()
            if k >= warm:
                evs[k - warm][1].record()
        pending.pop().current_stream_wait()
        torch.cuda.synchronize()
        return sorted(a.elapsed_time(b) * 1e3 for a, b in evs)

    t_layout = timed_layout(n_k)
    # what a pair of events costs by itself on this stream (nothing between them), to take off the layout figure
    t_events = timed(lambda: None, n_k)
    avg = lambda v: sum(v) / len(v)  # noqa: E731
    med = lambda v: v[len(v) // 2]  # noqa: E731
    us_scatter = med(t_scatter)

    def host_issue_us(n):
        # What the calls cost on the host: a dispatch without the host's wait for the counts and a combine are only
        # enqueued (outputs at their worst-case sizes), nothing waits for the GPU inside the bracket.
        r0, _, rw0, h0, _ = buf.dispatch(xg, topk_idx=tg, topk_weights=wg, do_cpu_sync=False, **kw)
        y_ws = torch.empty(((r0[0] if fp8 else r0).size(0), H), dtype=torch.bfloat16, device=dev)
        del r0, rw0, h0
        best = None
        for _ in range(3):
            torch.cuda.synchronize()
            t_start = time.perf_counter()
            for _ in range(n):
                r1, _, rw1, h1, _ = buf.dispatch(xg, topk_idx=tg, topk_weights=wg, do_cpu_sync=False, **kw)
                buf.combine(y_ws, h1, topk_weights=rw1)
            t_host = (time.perf_counter() - t_start) * 1e6 / n
            best = t_host if best is None else min(best, t_host)
        torch.cuda.synchronize()
        return best

    us_host = host_issue_us(20 if T * H >= (1 << 24) else 200)
    traffic, traffic_source = measured_traffic(args.workload) if not args.no_cpu_sync else ({}, 'not the profiled configuration')

    def roof(name, nbytes, samples):
        us = med(samples)
        gbs = nbytes / us / 1e3
        return {'kernel': name, 'bound': 'hbm', 'achieved': round(gbs, 1), 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
                'frac': round(gbs / HBM_PEAK_GBS, 4), 'traffic': traffic.get(name), 'us': round(us, 2),
                'us_mean': round(avg(samples), 2), 'us_min': round(samples[0], 2), 'samples': len(samples),
                'bytes': nbytes}

    scatter_name = 'ep_scatter_quant' if fused else 'ep_scatter_copy'
    kernels = [roof(scatter_name, b_d, t_scatter), roof(f'ep_combine_k{K}', b_c, t_combine)]
    for k in kernels:
        k['sampled'] = 'isolated launches' + ('' if args.no_flush else ', caches flushed before each')
    kernels[0]['sampled'] += '; the epilogue of a deferred non-cached dispatch (its layout kernels in front of the bracket)'
    kernels[0]['us_cached_replay'] = round(med(t_scatter_cached), 2)
    # The dominant kernel, priced on its launches inside the timed region (event to event on the launch
    # stream: the kernel plus the gap to its predecessor).
    if loop_combine is not None:
        dominant = roof(f'ep_combine_k{K}', b_c, loop_combine)
        us_dispatch, us_combine = med(loop_dispatch), med(loop_combine)
    else:
        dominant = max(kernels, key=lambda k: k['us'])
        us_dispatch, us_combine = med(t_dispatch_full), med(t_combine)
    roofline = {k: dominant[k] for k in ('bound', 'achieved', 'peak', 'unit', 'frac', 'traffic')}
    roofline.update({
        'kernel': dominant['kernel'], 'traffic_source': traffic_source,
        # both kernels of the path, each alone (median of the isolated, flushed launches), as fractions of 8 TB/s
        'dispatch_kernel': scatter_name, 'dispatch_frac': kernels[0]['frac'], 'dispatch_achieved': kernels[0]['achieved'],
        'dispatch_traffic': kernels[0]['traffic'],
        'dispatch_frac_incl_zero_padding': round((b_d + pad_bytes) / us_scatter / 1e3 / HBM_PEAK_GBS, 4),
        'combine_kernel': kernels[1]['kernel'], 'combine_frac': kernels[1]['frac'], 'combine_achieved': kernels[1]['achieved'],
        'combine_traffic': kernels[1]['traffic'],
        # the dispatch phase inside the timed region: layout kernels + copy kernel (+ the gaps between them)
        'dispatch_phase_frac': round(b_d / us_dispatch / 1e3 / HBM_PEAK_GBS, 4)})
    out = {
        'metric': 'dispatch & combine GB/s + % of HBM peak, 16384 tok x7168, top-6/256, FP8/BF16',
        'value': round((b_d + b_c) / ms_per_step / 1e6, 1), 'unit': 'GB/s',
        'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': round(ms_per_step, 4),
        'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'fp8_e4m3+bf16 payload, fp32 accumulate' if fp8 else 'bf16 payload, fp32 accumulate',
        'data': 'synthetic',
        'config': {'workload': args.workload, 'tokens': T, 'hidden': H, 'experts': E, 'topk': K,
                   'expert_alignment': A, 'partitions': 1, 'dispatch': 'fused bf16->fp8 e4m3 + per-128 fp32 scales'
                   if fused else ('fp8 e4m3 rows + per-128 fp32 scales quantised by the caller' if fp8 else 'bf16'), 'combine': 'bf16, fp32 accumulate, weights carried back, no bias',
                   'do_zero_padding': True, 'do_cpu_sync': not args.no_cpu_sync, 'hip_graph': bool(args.graph),
                   'cache_flush_between_kernel_samples': not args.no_flush,
                   'num_valid_rows': n_valid, 'num_expanded_rows': n_exp_exact},
        'roofline': roofline,
        'kernels': kernels,
        'phases': {
            'measured': 'inside the timed region, medians' if loop_combine is not None else 'isolated launches, medians',
            'dispatch_us': round(us_dispatch, 2),
            # the layout kernels alone: events around a deferred dispatch launch (flushed caches) minus what an empty
            # pair of events measures; the host's read of the counts runs while the copy kernel does and adds nothing
            'dispatch_layout_and_host_sync_us': round(med(t_layout) - med(t_events), 2),
            'dispatch_layout_events_raw_us': round(med(t_layout), 2), 'empty_event_pair_us': round(med(t_events), 2),
            'dispatch_copy_kernel_in_loop_us': round(us_dispatch - (med(t_layout) - med(t_events)), 2),
            'dispatch_isolated_flushed_us': round(med(t_dispatch_full), 2),
            'dispatch_gbs': round(b_d / us_dispatch / 1e3, 1), 'dispatch_frac_hbm': round(b_d / us_dispatch / 1e3 / HBM_PEAK_GBS, 4),
            'combine_us': round(us_combine, 2), 'combine_gbs': round(b_c / us_combine / 1e3, 1),
            'combine_frac_hbm': round(b_c / us_combine / 1e3 / HBM_PEAK_GBS, 4),
            # host time of the two calls (enqueue only: dispatch without host sync + combine; best of three loops)
            'host_us': round(us_host, 2),
            'dispatch_bytes': b_d, 'combine_bytes': b_c, 'zero_padding_bytes_not_counted': pad_bytes,
            'scatter_gbs_incl_padding': round((b_d + pad_bytes) / us_scatter / 1e3, 1),
        },
    }
    if fused:
        # the ceiling of the copy kernel's formulation, from calibration kernels run here (outputs of the first
        # dispatch serve as their scratch outputs)
        import ep_calib
        ep_calib.init()
        cargs, keep = calib_scatter_args(ep_calib, xg, wg, handle, recv[0], recv[1], recv_w, T, H, K, E, A)
        roofline['dispatch_ceiling'] = dispatch_ceiling(ep_calib, timed, n_k, cargs, us_scatter)
        if K == 6:
            # the same for the combine kernel (isolated flushed median against its two streams alone)
            blocks_per_cu = 3 if args.combine_blocks_per_cu is None or args.combine_blocks_per_cu < 0 else args.combine_blocks_per_cu
            cx = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
            cw = torch.empty((T, K), dtype=torch.float32, device=dev)
            ccargs, ckeep = calib_combine_args(ep_calib, y, recv_w, handle, cx, cw, T, H, K, E, blocks_per_cu)
            roofline['combine_ceiling'] = combine_ceiling(ep_calib, timed, n_k, ccargs, med(t_combine))
            del ckeep, cx, cw
        if args.calibrate_write:
            out['write_calibration'] = calibrate_write(ep_calib, timed, n_k, cargs, T, H, K, n_valid, n_recv, pad_bytes,
                                                       dev, us_scatter, handle.recv_src_metadata)
        del keep
    if not args.no_cpu_baseline:
        out['cpu_baseline'] = cpu_baseline(H, E, K, A, fp8, min(args.cpu_sample_tokens, T))
    buf.destroy()
    print(json.dumps(out))


if __name__ == '__main__':
    main()
