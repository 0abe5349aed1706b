"""Seeded input generators shared by the CPU and GPU tests (all data is made on the CPU)."""
import numpy as np
import torch


def bf16_from_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def make_tokens(T, H, seed=0, outliers=False):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((T, H), generator=g, dtype=torch.float32)
    if outliers:
        x[torch.rand((T, H), generator=g) < 1e-3] *= 50
    return x.to(torch.bfloat16)


def make_routing(T, E, K, seed=0, masked=0.0, zipf=None):
    """topk_idx [T,K] int64 and fp32 softmax gate weights; Zipf(s) popularity when `zipf` is set;
    a fraction `masked` of slots set to -1 with weight 0."""
    g = torch.Generator().manual_seed(seed + 7919)
    if zipf is None:
        logits = torch.randn((T, E), generator=g, dtype=torch.float32)
        val, idx = torch.topk(logits, K, dim=-1, sorted=True)
        w = torch.softmax(val, dim=-1)
    else:
        p = (torch.arange(E, dtype=torch.float64) + 1) ** (-zipf)
        idx = torch.multinomial((p / p.sum()).expand(T, E), K, replacement=False, generator=g)
        w = torch.softmax(torch.randn((T, K), generator=g), dim=-1)
    idx = idx.to(torch.int64)
    if masked > 0:
        m = torch.rand((T, K), generator=g) < masked
        idx = idx.masked_fill(m, -1)
        w = w.masked_fill(m, 0.0)
    return idx.contiguous(), w.contiguous().float()
