"""CPU-only checks of the native library: it loads, exports every symbol the C header declares,
and its host-side pieces (size calculators, the integer e4m3fn conversion) agree with the oracle
and with torch.  No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from oracle import ep_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, 'include', 'deep_ep_hip.h')
LIB = os.path.join(ROOT, 'deepep-ascend_amd', 'deep_ep', 'lib', 'libdeep_ep_hip.so')


@pytest.fixture(scope='module')
def de():
    if not os.path.exists(LIB):
        import __graft_entry__
        __graft_entry__.build()
    import deep_ep
    return deep_ep


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(ep_[a-z0-9_]+)\s*\(', text)))


def test_library_exports_every_declared_symbol(de):
    lib = ctypes.CDLL(LIB)
    names = declared_symbols()
    assert len(names) >= 18
    for n in names:
        assert hasattr(lib, n), n


def test_code_object_is_built_for_gfx950(de):
    path = os.path.join(os.path.dirname(LIB), 'ep_kernels.hsaco')
    blob = open(path, 'rb').read()
    assert blob[:4] == b'\x7fELF' or blob.startswith(b'__CLANG_OFFLOAD_BUNDLE__')
    for k in (b'ep_layout_count', b'ep_layout_scan', b'ep_layout_assign', b'ep_scatter_copy', b'ep_scatter_quant',
              b'ep_combine_k6', b'ep_combine_generic', b'gfx950'):
        assert k in blob, k


def test_code_object_has_every_instance_of_the_slot_assignment(de):
    blob = open(os.path.join(os.path.dirname(LIB), 'ep_kernels.hsaco'), 'rb').read()
    for k in (b'ep_layout_assign_fold', b'ep_layout_assign_recv', b'ep_layout_assign_fold_recv'):
        assert k in blob, k


def test_slot_assignment_keeps_its_count_rows_in_flight(de, tmp_path):
    """Two properties of the compiled kernels that the timings rest on and that a source change can lose without any
    result changing, read from the compiler's assembly of the committed sources (same flags as the build):
    no kernel reserves a private segment (no spills: the library's entry point for callers that cannot allocate must not
    make the runtime set up scratch memory), and in the slot assignment that sums the block counts itself the 22 row
    loads issued at the top are still in flight behind the staging of the ids and while the ids are counted per wave (the
    compiler's wait-count pass merges the paths through the kernel: a wait for fewer outstanding loads there means that
    the ids, or their counting, wait for the rows again)."""
    import shutil
    import subprocess
    from deep_ep import _build
    if shutil.which(_build.HIPCC) is None and not os.path.exists(_build.HIPCC):
        pytest.skip('no hipcc here')
    out = tmp_path / 'ep_kernels.s'
    flags = [f for f in _build.DEVICE_FLAGS if f != '--genco']
    subprocess.check_call([_build.HIPCC, *flags, '--cuda-device-only', '-S', '-o', str(out),
                           os.path.join(_build.CSRC, 'ep_kernels.hip')], stderr=subprocess.DEVNULL)
    text = out.read_text()
    sizes = re.findall(r'\.amdhsa_private_segment_fixed_size (\d+)', text)
    assert len(sizes) >= 30 and set(sizes) == {'0'}, sizes
    body = text[text.index('\nep_layout_assign_fold:'):]
    body = body[:body.index('.end_amdhsa_kernel')]
    # in the order of the listing: ..., the ids waited for with the 22 row loads left outstanding, the barrier behind their
    # staging, and the next wait for a load is the one for the first row, where the rows are summed
    marks = []
    for line in body.splitlines():
        line = line.strip()
        m = re.match(r's_waitcnt.*vmcnt\((\d+)\)', line)
        if m:
            marks.append(int(m.group(1)))
        elif line.startswith('s_barrier'):
            marks.append('barrier')
    assert any(marks[i:i + 3] == [22, 'barrier', 21] for i in range(len(marks))), marks


def test_size_calculators_match_oracle(de):
    C = de._C
    for (R, T, H, K, fp8) in [(1, 16384, 7168, 6, False), (1, 16384, 7168, 6, True), (32, 16384, 7168, 6, True),
                              (8, 4096, 7168, 8, False), (2, 128, 256, 0, False), (4, 7, 2048, 3, True)]:
        assert C.calculate_ep_buffer_size(R, T, H, K, fp8) == O.calculate_buffer_size(R, T, H, K, fp8)
    assert C.get_dispatch_buffer_size(16384, 7168, 112, 6, 1, 32) == 32 * 16384 * 7488
    assert C.get_combine_buffer_size(32, 16384, 7168, 6) == 6 * 16384 * 14368
    assert C.get_combine_buffer_size(2, 100, 256, 6) == 2 * 100 * (512 + 32)
    assert (C.get_num_allocation_alignment(), C.get_num_tma_alignment(), C.get_num_rdma_alignment()) == (2097152, 32, 32)
    assert de.topk_idx_t == torch.int64
    with pytest.raises(C.EPException, match=r'Assertion exception \(ep_runtime.cpp:\d+\): hidden > 0'):
        C.calculate_ep_buffer_size(1, 1, 0, 1, False)


def test_integer_e4m3fn_conversion_matches_torch(de):
    C = de._C
    # all BF16 values widened to fp32 (the quantiser's inputs) times assorted scales, plus dense sweeps
    allbf = torch.from_numpy((np.arange(65536, dtype=np.uint32) << 16).view(np.float32).copy())
    for scale in (1.0, 448.0 / 3.0, 448.0 / 0.0123, 2.0 ** -7, 448.0 / 1e-4, 0.37):
        f = allbf * scale
        f = f[torch.isfinite(f)]
        assert torch.equal(C.host_f32_to_e4m3fn(f), f.to(torch.float8_e4m3fn).view(torch.uint8)), scale
    g = torch.Generator().manual_seed(0)
    bits = torch.randint(0, 2 ** 31 - 1, (4_000_000,), generator=g, dtype=torch.int64).to(torch.int32)
    f = bits.view(torch.float32)
    f = torch.cat([f, -f])
    f = f[torch.isfinite(f)]
    assert torch.equal(C.host_f32_to_e4m3fn(f), f.to(torch.float8_e4m3fn).view(torch.uint8))
    # every fp32 value in [2^-12, 512): all rounding boundaries of the format, strided
    lo, hi = np.float32(2.0 ** -12).view(np.uint32), np.float32(512.0).view(np.uint32)
    dense = torch.from_numpy(np.arange(lo, hi, 37, dtype=np.uint32).view(np.float32).copy())
    assert torch.equal(C.host_f32_to_e4m3fn(dense), dense.to(torch.float8_e4m3fn).view(torch.uint8))
    # ties exactly half way between neighbouring codes
    codes = torch.arange(0, 0x7F, dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    mids = (codes[:-1] + codes[1:]) / 2
    assert torch.equal(C.host_f32_to_e4m3fn(mids), mids.to(torch.float8_e4m3fn).view(torch.uint8))


def test_no_gpu_means_loud_failure(de):
    if torch.cuda.is_available():
        pytest.skip('GPU present')
    with pytest.raises(de._C.EPException, match='needs a GPU'):
        de.EPBuffer(de.LocalGroup(), num_max_tokens_per_rank=8, hidden=64, num_topk=2)


def test_event_overlap_runs_hook_once(de):
    class FakeEvent:
        waits = 0

        def current_stream_wait(self):
            FakeEvent.waits += 1

    ev = de.EventOverlap(FakeEvent())
    calls = []
    ev.register_hook_after_wait(lambda: calls.append(1) or 'result')
    with pytest.raises(AssertionError):
        ev.register_hook_after_wait(lambda: None)
    assert ev.current_stream_wait() == 'result'
    assert ev.wait() is None and calls == [1] and FakeEvent.waits == 2
    with ev(release_handle=True):
        pass
    assert ev.event is None and FakeEvent.waits == 3


def test_buffer_allocator_plans_aligned_meta_tensors(de):
    plan = de.BufferAllocator()
    a = plan.allocate((3, 5), torch.float32)
    b = plan.allocate((7,), torch.bfloat16)
    assert a.is_meta and b.is_meta
    assert [off for _, off in plan.allocations] == [0, 2097152]
    assert plan.num_bytes == 2 * 2097152


def test_python_quantiser_matches_oracle(de):
    g = torch.Generator().manual_seed(3)
    x = (torch.randn((32, 384), generator=g) * 3).to(torch.bfloat16)
    q, s = de.utils.math.per_token_cast_to_fp8(x)
    oq, os_ = O.quantise(x)
    assert torch.equal(q.view(torch.uint8), oq) and torch.equal(s, os_)
    back = de.utils.math.per_token_cast_back(q, s)
    assert (back.float() - x.float()).abs().max() <= 0.07 * x.float().abs().max()


def test_ctypes_structs_match_the_header(de, tmp_path):
    """The Python binding restates the argument structs of the header: compile the header with gcc and
    compare sizes and the offsets of the trailing fields."""
    import subprocess
    src = tmp_path / 'abi.c'
    src.write_text('''
#include <stdio.h>
#include <stddef.h>
#include "deep_ep_hip.h"
int main(void) {
    printf("%zu %zu %zu %zu\\n", sizeof(ep_tensor_t), sizeof(ep_dispatch_args_t),
           sizeof(ep_dispatch_epilogue_args_t), sizeof(ep_combine_args_t));
    printf("%zu %zu %zu %zu\\n", offsetof(ep_dispatch_args_t, stream), offsetof(ep_dispatch_args_t, fused_fp8_quant),
           offsetof(ep_dispatch_epilogue_args_t, stream), offsetof(ep_dispatch_epilogue_args_t, recv_sf_layout));
    printf("%zu %zu\\n", offsetof(ep_combine_args_t, stream), offsetof(ep_combine_args_t, apply_weights));
    printf("%zu %zu %zu\\n", sizeof(ep_dispatch_recv_args_t), offsetof(ep_dispatch_recv_args_t, stream),
           offsetof(ep_dispatch_recv_args_t, hidden_bytes));
    printf("%zu %zu\\n", offsetof(ep_dispatch_epilogue_args_t, dispatch_stamp),
           offsetof(ep_dispatch_recv_args_t, dispatch_stamp));
    return 0;
}
''')
    exe = tmp_path / 'abi'
    subprocess.run(['gcc', '-I', os.path.join(ROOT, 'include'), '-o', str(exe), str(src)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    C = de._C
    got = [ctypes.sizeof(C._Tensor), ctypes.sizeof(C._DispatchArgs), ctypes.sizeof(C._DispatchEpilogueArgs),
           ctypes.sizeof(C._CombineArgs),
           C._DispatchArgs.stream.offset, C._DispatchArgs.fused_fp8_quant.offset,
           C._DispatchEpilogueArgs.stream.offset, C._DispatchEpilogueArgs.recv_sf_layout.offset,
           C._CombineArgs.stream.offset, C._CombineArgs.apply_weights.offset,
           ctypes.sizeof(C._DispatchRecvArgs), C._DispatchRecvArgs.stream.offset,
           C._DispatchRecvArgs.hidden_bytes.offset,
           C._DispatchEpilogueArgs.dispatch_stamp.offset, C._DispatchRecvArgs.dispatch_stamp.offset]
    assert got == [int(v) for v in out]


def test_bench_byte_formulas_give_the_headline_figures():
    """The algorithmic bytes bench.py prices the kernels with, at the headline configuration
    (16384 x 7168, top-6, every selection valid): 14 336 B read + 6 x 7396 B written per token plus
    metadata for the fused FP8 dispatch, 6 x 14 336 B read + 14 336 B written for the combine."""
    import importlib.util
    spec = importlib.util.spec_from_file_location('bench_module', os.path.join(ROOT, 'bench.py'))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    T, H, K = 16384, 7168, 6
    assert bench.dispatch_bytes(T, H, K, T * K, T, True, True) == 964427776
    assert bench.combine_bytes(T, H, K, T * K, T, 0, True) == 1646264320
    assert bench.dispatch_bytes(4096, H, 8, 4096 * 8, 4096, False, False) == 529432576      # BF16 top-8
    assert bench.WORKLOADS['c3_headline'] == (T, H, 256, K, 128, True)


def test_committed_traffic_summary_belongs_to_the_kernel_sources():
    """bench.py reports HBM traffic from the committed counter summary only while that summary was taken from
    the kernel sources in the tree (its kernel_source_sha256 line): a kernel change needs a fresh counter run."""
    import importlib.util
    spec = importlib.util.spec_from_file_location('bench_module_traffic', os.path.join(ROOT, 'bench.py'))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    traffic, source = bench.measured_traffic('c3_headline')
    assert source.endswith('headline_dispatch_combine_hbm_traffic.txt'), source
    # measured traffic = algorithmic bytes (+ the zero padding the copy kernel also writes), nothing re-read
    assert 1.0 <= traffic['ep_scatter_quant'] / (964427776 + 115495936) < 1.02
    assert 1.0 <= traffic['ep_combine_k6'] / 1646264320 < 1.02


def test_bench_refuses_more_than_one_gpu():
    """One GPU's share is all this path has: asked for more, bench.py says so and exits with a usage error."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, 'bench.py'), '--gpus', '2'], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 2
    assert 'one GPU' in r.stderr and r.stdout.strip() == ''


def test_calibration_rig_is_a_library_of_its_own(de):
    """The benchmarks' calibration kernels live in their own library and code object: the product exports and
    ships none of them, and the calibration library exports what its header declares."""
    calib_dir = os.path.join(ROOT, 'deepep-ascend_amd', 'ep_calib', 'lib')
    text = re.sub(r'/\*.*?\*/', '', open(os.path.join(ROOT, 'include', 'deep_ep_calib.h')).read(), flags=re.S)
    names = sorted(set(re.findall(r'\b(ep_calib_[a-z0-9_]+)\s*\(', text)))
    assert len(names) >= 6
    calib = ctypes.CDLL(os.path.join(calib_dir, 'libdeep_ep_calib.so'))
    product = ctypes.CDLL(LIB)
    for n in names:
        assert hasattr(calib, n), n
        assert not hasattr(product, n), n
    for gone in ('ep_calibrate_fill', 'ep_set_calibration_stores_only'):
        assert not hasattr(product, gone), gone
    blob = open(os.path.join(os.path.dirname(LIB), 'ep_kernels.hsaco'), 'rb').read()
    assert b'ep_calib' not in blob and b'stores_only' not in blob
    cblob = open(os.path.join(calib_dir, 'ep_calib.hsaco'), 'rb').read()
    for k in (b'ep_calib_fill', b'ep_calib_fronts', b'ep_calib_mixed', b'ep_calib_scatter_stores_only', b'ep_calib_read_rows',
              b'ep_calib_ordered_steered', b'ep_calib_copy_ordered_flat', b'gfx950'):
        assert k in cblob, k
