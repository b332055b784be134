"""e4m3fn block quantisers and the synthetic inputs of the benchmark configurations.

The reference receives its operands already quantised from the harness
(1-amd-fp8-mm/0-amd-fp8-mm-new-begins.py:66-77); this module produces tensors of exactly those shapes,
dtypes and K-major strides from fp32 data, so that tests, the smoke run and the benchmark all feed
``custom_kernel`` what the harness would.

Quantisation rule (per block): scale = max(|x|)/448 stored as fp32, q = x/scale rounded to e4m3fn
(round-to-nearest-even, clamped to +-448 first because torch's cast does not saturate).  A is
quantised per 1x128 block (one row, 128 consecutive k), B per 128x128 block.
"""
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

FP8_MAX = 448.0
BLOCK = 128
_TINY = 1e-12     # all-zero block: any positive scale works, the codes are all zero


def _kmajor(t: torch.Tensor) -> torch.Tensor:
    """Return a [rows, cols] view with stride (1, rows): storage holds the transpose contiguously."""
    return t.t().contiguous().t()


def quantize_a(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp32 [M, K] -> (a float8_e4m3fn [M, K] stride (1, M), a_scale fp32 [M, K/128] stride (1, M))."""
    m, k = x.shape
    assert k % BLOCK == 0
    xb = x.float().reshape(m, k // BLOCK, BLOCK)
    scale = (xb.abs().amax(dim=2) / FP8_MAX).clamp_min(_TINY)
    q = (xb / scale.unsqueeze(2)).clamp_(-FP8_MAX, FP8_MAX).reshape(m, k).to(torch.float8_e4m3fn)
    return _kmajor(q), _kmajor(scale)


def quantize_b(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp32 [N, K] -> (b float8_e4m3fn [N, K] stride (1, N), b_scale fp32 [ceil(N/128), K/128] stride (1, NB)).

    A partial last block of rows (N not a multiple of 128) takes its amax over the rows that exist.
    """
    n, k = w.shape
    assert k % BLOCK == 0
    nb, kb = (n + BLOCK - 1) // BLOCK, k // BLOCK
    wp = w.float()
    if nb * BLOCK != n:
        wp = torch.cat([wp, wp.new_zeros(nb * BLOCK - n, k)], dim=0)
    wb = wp.reshape(nb, BLOCK, kb, BLOCK)
    scale = (wb.abs().amax(dim=(1, 3)) / FP8_MAX).clamp_min(_TINY)           # [nb, kb]
    q = (wb / scale[:, None, :, None]).clamp_(-FP8_MAX, FP8_MAX).reshape(nb * BLOCK, k)[:n]
    return _kmajor(q.to(torch.float8_e4m3fn)), _kmajor(scale)


@dataclass(frozen=True)
class Config:
    """One benchmark configuration (sizes, input distributions and seed)."""
    name: str
    m: int            # rows of A (grouped: tokens before routing)
    n: int
    k: int
    a_outlier_frac: float = 0.0   # fraction of A entries multiplied by a_outlier_mul
    a_outlier_mul: float = 1.0
    b_std: float = 1.0
    experts: int = 0              # > 0: grouped, every token routed to `topk` distinct experts
    topk: int = 0
    seed: int = 0


CONFIGS = (
    Config("cfg1_plumbing_256x512x1024", 256, 512, 1024, seed=20251),
    Config("cfg2_square_4096", 4096, 4096, 4096, seed=20252),
    Config("cfg3_qa_kva_4096x2112x7168", 4096, 2112, 7168, a_outlier_frac=0.01, a_outlier_mul=20.0, b_std=0.02, seed=20253),
    Config("cfg4_skinny_64x18432x7168", 64, 18432, 7168, b_std=0.02, seed=20254),
    Config("cfg5_grouped_moe_32x4096x7168", 4096, 4096, 7168, b_std=0.02, experts=32, topk=8, seed=20255),
)


def _draw_a(cfg: Config, m: int, gen: torch.Generator) -> torch.Tensor:
    x = torch.randn(m, cfg.k, generator=gen, dtype=torch.float32)
    if cfg.a_outlier_frac > 0:
        mask = torch.rand(m, cfg.k, generator=gen) < cfg.a_outlier_frac
        x = torch.where(mask, x * cfg.a_outlier_mul, x)
    return x


def make_dense(cfg: Config, device: Optional[torch.device] = None, m: Optional[int] = None,
               n: Optional[int] = None, k: Optional[int] = None):
    """Inputs of a dense configuration as the 5-tuple ``custom_kernel`` takes (c is zero-filled).

    ``m``/``n``/``k`` shrink the shape (same distributions, same seed) for cases a CPU oracle must
    finish quickly.  Tensors are generated on the CPU with a seeded generator, then moved.
    """
    assert cfg.experts == 0
    if k is not None or n is not None or m is not None:
        cfg = Config(cfg.name, m or cfg.m, n or cfg.n, k or cfg.k, cfg.a_outlier_frac, cfg.a_outlier_mul,
                     cfg.b_std, 0, 0, cfg.seed)
    gen = torch.Generator().manual_seed(cfg.seed)
    a, a_scale = quantize_a(_draw_a(cfg, cfg.m, gen))
    w = torch.randn(cfg.n, cfg.k, generator=gen, dtype=torch.float32) * cfg.b_std
    b, b_scale = quantize_b(w)
    c = torch.zeros(cfg.m, cfg.n, dtype=torch.bfloat16)
    data = (a, b, a_scale, b_scale, c)
    if device is not None:
        data = tuple(_to_device(t, device) for t in data)
    return data


def _to_device(t: torch.Tensor, device) -> torch.Tensor:
    """Move a tensor keeping its strides (``.to`` preserves dense non-overlapping layouts)."""
    out = t.to(device)
    assert out.stride() == t.stride()
    return out


def make_grouped(cfg: Config, device: Optional[torch.device] = None, tokens: Optional[int] = None,
                 n: Optional[int] = None, k: Optional[int] = None, experts: Optional[int] = None,
                 topk: Optional[int] = None):
    """Inputs of the grouped configuration: ``(a, b, a_scale, b_scale, row_offsets, c)``.

    Tokens are quantised per 1x128 before routing; every token goes to ``topk`` distinct experts
    chosen uniformly (``torch.rand(tokens, experts).topk(topk)``); rows are gathered
    expert-contiguous, stable by token id.  ``row_offsets`` is int32 [experts+1].
    """
    e = experts or cfg.experts
    tk = topk or cfg.topk
    t_, n_, k_ = tokens or cfg.m, n or cfg.n, k or cfg.k
    gen = torch.Generator().manual_seed(cfg.seed)
    x = torch.randn(t_, k_, generator=gen, dtype=torch.float32)
    qa, qs = quantize_a(x)                                       # [T, K] / [T, K/128], K-major views
    route = torch.rand(t_, e, generator=gen).topk(tk, dim=1).indices      # [T, topk]
    token_ids = torch.arange(t_).repeat_interleave(tk)
    expert_ids = route.reshape(-1)
    order = torch.sort(expert_ids * t_ + token_ids).indices                # by expert, then token id
    perm = token_ids[order]
    counts = torch.bincount(expert_ids, minlength=e)
    row_offsets = torch.zeros(e + 1, dtype=torch.int32)
    row_offsets[1:] = torch.cumsum(counts, 0).to(torch.int32)
    rows = int(row_offsets[-1])
    # gather rows in storage order ([K, rows]) so the result is K-major without a second copy
    a = qa.t().view(torch.uint8)[:, perm].contiguous().view(torch.float8_e4m3fn).t()
    a_scale = qs.t()[:, perm].contiguous().t()
    nb, kb = (n_ + BLOCK - 1) // BLOCK, k_ // BLOCK
    b_store = torch.empty(e, k_, n_, dtype=torch.float8_e4m3fn)            # storage [E][K][N]
    bs_store = torch.empty(e, kb, nb, dtype=torch.float32)
    for x_ in range(e):                                                    # one expert at a time: bounds fp32 memory
        w = torch.randn(n_, k_, generator=gen, dtype=torch.float32) * cfg.b_std
        qb, sb = quantize_b(w)
        b_store[x_] = qb.t()
        bs_store[x_] = sb.t()
    b = b_store.transpose(1, 2)                                            # [E, N, K], each expert K-major
    b_scale = bs_store.transpose(1, 2)
    c = torch.zeros(rows, n_, dtype=torch.bfloat16)
    data = (a, b, a_scale, b_scale, row_offsets, c)
    if device is not None:
        data = tuple(_to_device(t, device) for t in data)
    return data
