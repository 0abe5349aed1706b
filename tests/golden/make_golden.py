"""Writes the golden vectors under tests/golden/ from the reference's own pure-torch helpers.

Runs only where the reference checkout exists (the build container); the vectors it writes are
committed, the reference is not.  Three reference functions are exercised, each loaded by file
path because the reference package itself needs its unbuilt native module to import:

* deep_ep/utils/math.py  per_token_cast_to_fp8   -> quantiser vectors
* deep_ep/utils/refs.py  combine                 -> combine vectors (world sizes 1, 2 and 4)
* deep_ep/utils/refs.py  dispatch                -> dispatch ordering/masking vectors (world size 2)

refs.py asks torch.distributed for rank / world size, so those cases run under a gloo group on
127.0.0.1 with CPU tensors.

Usage:  python tests/golden/make_golden.py [/root/reference]
"""
import importlib
import os
import sys
import types

import numpy as np
import torch
import torch.distributed as dist
import torch.multiprocessing as mp

HERE = os.path.dirname(os.path.abspath(__file__))


def load_ref_utils(ref_root: str):
    pkg = types.ModuleType('ref_deep_ep_utils')
    pkg.__path__ = [os.path.join(ref_root, 'deep_ep', 'utils')]
    sys.modules['ref_deep_ep_utils'] = pkg
    math_mod = importlib.import_module('ref_deep_ep_utils.math')
    refs_mod = importlib.import_module('ref_deep_ep_utils.refs')
    return math_mod, refs_mod


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def quant_inputs():
    g = torch.Generator().manual_seed(1234)
    cases = {}
    x = torch.randn((8, 256), generator=g)
    cases['randn_8x256'] = x.to(torch.bfloat16)
    x = torch.randn((6, 384), generator=g)
    x[torch.rand((6, 384), generator=g) < 0.02] *= 50
    cases['outliers_6x384'] = x.to(torch.bfloat16)
    x = torch.randn((5, 200), generator=g) * 1e-3          # hidden not a multiple of 128
    cases['small_5x200'] = x.to(torch.bfloat16)
    x = torch.zeros((3, 256))
    x[1, :128] = torch.randn(128, generator=g) * 1e-6      # below the 1e-4 clamp
    x[2, 5] = 448.0
    x[2, 130] = -3.0e4
    cases['edge_3x256'] = x.to(torch.bfloat16)
    return cases


def make_quant(math_mod):
    out = {}
    for name, x in quant_inputs().items():
        q, s = math_mod.per_token_cast_to_fp8(x)
        out[name + '.x'] = bf16_bits(x)
        out[name + '.q'] = q.view(torch.uint8).numpy().copy()
        out[name + '.s'] = s.contiguous().numpy().copy()
    np.savez_compressed(os.path.join(HERE, 'quant_golden.npz'), **out)
    print('quant_golden.npz:', sorted(out))


def combine_case(seed: int, T: int, K: int, E: int, H: int, masked: float, nbias: int):
    g = torch.Generator().manual_seed(seed)
    y = (torch.randn((T, K, H), generator=g) * 3).to(torch.bfloat16)
    scores = torch.randn((T, E), generator=g)
    topk_idx = torch.topk(scores, K, dim=-1, sorted=False).indices.to(torch.int64)
    if masked > 0:
        topk_idx[torch.rand((T, K), generator=g) < masked] = -1
    bias = tuple(torch.randn((T, H), generator=g).to(torch.bfloat16) for _ in range(nbias))
    return y, topk_idx, bias


COMBINE_CASES = [  # seed, T, K, E, H, masked, nbias
    (1, 16, 4, 8, 64, 0.0, 0),
    (2, 16, 4, 8, 64, 0.2, 1),
    (3, 12, 6, 16, 32, 0.1, 2),
    (4, 9, 2, 8, 32, 0.5, 0),
    (5, 10, 8, 8, 32, 0.0, 2),
]


def _worker(rank: int, world: int, port: int, ref_root: str, what: str):
    dist.init_process_group('gloo', init_method=f'tcp://127.0.0.1:{port}', world_size=world, rank=rank)
    _, refs_mod = load_ref_utils(ref_root)
    out = {}
    if what == 'combine':
        for ci, (seed, T, K, E, H, masked, nbias) in enumerate(COMBINE_CASES):
            y, topk_idx, bias = combine_case(seed, T, K, E, H, masked, nbias)
            y_in = y.clone()
            y_in[topk_idx == -1] = 0                       # as tests/ep/test_ep.py:301
            b = None if nbias == 0 else (bias[0] if nbias == 1 else bias)
            res = refs_mod.combine(y_in.clone(), topk_idx, E, b, reduce_in_local=True)
            p = f'w{world}.c{ci}.'
            out[p + 'y'] = bf16_bits(y)
            out[p + 'topk_idx'] = topk_idx.numpy().copy()
            for bi, bt in enumerate(bias):
                out[p + f'bias{bi}'] = bf16_bits(bt)
            out[p + 'cfg'] = np.array([T, K, E, H, nbias, world], dtype=np.int64)
            out[p + 'out'] = bf16_bits(res)
        if rank == 0:
            np.savez_compressed(os.path.join(HERE, f'combine_golden_w{world}.npz'), **out)
            print(f'combine_golden_w{world}.npz: {len(out)} arrays')
    else:
        T, K, E, H, maxT = 12 - rank, 3, 8, 16, 12
        g = torch.Generator().manual_seed(100 + rank)
        x = torch.randn((T, H), generator=g).to(torch.bfloat16)
        scores = torch.randn((T, E), generator=g)
        w, idx = torch.topk(scores, K, dim=-1, sorted=False)
        idx = idx.to(torch.int64)
        idx[torch.rand((T, K), generator=g) < 0.15] = -1
        w = w.masked_fill(idx < 0, 0)
        rx, ridx, rw, rsrc, rcnt = refs_mod.dispatch(x, idx, w, maxT, E)
        gathered = [None] * world
        mine = dict(x=bf16_bits(x), topk_idx=idx.numpy().copy(), topk_weights=w.numpy().copy(),
                    recv_x=bf16_bits(rx), recv_topk_idx=ridx.numpy().copy(), recv_topk_weights=rw.numpy().copy(),
                    recv_src_token_idx=rsrc.numpy().copy(), num_recv_tokens_per_rank=rcnt.numpy().copy(),
                    cfg=np.array([T, K, E, H, maxT, world], dtype=np.int64))
        dist.all_gather_object(gathered, mine)
        if rank == 0:
            for r, d in enumerate(gathered):
                for k, v in d.items():
                    out[f'r{r}.{k}'] = v
            np.savez_compressed(os.path.join(HERE, f'dispatch_golden_w{world}.npz'), **out)
            print(f'dispatch_golden_w{world}.npz: {len(out)} arrays')
    dist.barrier()
    dist.destroy_process_group()


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else '/root/reference'
    math_mod, _ = load_ref_utils(ref_root)
    make_quant(math_mod)
    port = 29731
    for world in (1, 2, 4):
        mp.spawn(_worker, args=(world, port, ref_root, 'combine'), nprocs=world)
        port += 1
    mp.spawn(_worker, args=(2, port, ref_root, 'dispatch'), nprocs=2)


if __name__ == '__main__':
    main()
