"""Seeded synthetic inputs for the benchmark configurations (collider events, gated-delta operands).

All generators draw on the CPU with ``torch.Generator`` so that the same seed gives the same tensors on
every machine; the caller moves them to the GPU.
"""
import math

import torch

BARREL_RADII_MM = (32.0, 72.0, 116.0, 172.0, 260.0, 360.0, 500.0, 660.0, 820.0, 1020.0)


def collider_event(n_hits: int = 60000, seed: int = 0, feat_dim: int = 24):
    """One synthetic event: hits on 10 cylindrical barrel layers, eta ~ U(-4,4), phi ~ U(-pi,pi),
    z = r sinh(eta). Returns coords [N,4] = (eta, cos phi, sin phi, r/1020) fp32, feats [N,feat_dim] fp32
    ~ N(0,1) and the raw (r, eta, phi, z) columns [N,4]."""
    gen = torch.Generator().manual_seed(seed)
    radii = torch.tensor(BARREL_RADII_MM)
    layer = torch.randint(0, len(BARREL_RADII_MM), (n_hits,), generator=gen)
    r = radii[layer]
    eta = (torch.rand(n_hits, generator=gen) * 8.0 - 4.0)
    phi = (torch.rand(n_hits, generator=gen) * 2.0 - 1.0) * math.pi
    z = r * torch.sinh(eta)
    coords = torch.stack([eta, torch.cos(phi), torch.sin(phi), r / 1020.0], dim=1).float().contiguous()
    feats = torch.randn(n_hits, feat_dim, generator=gen)
    raw = torch.stack([r, eta, phi, z], dim=1)
    return coords, feats, raw


def lsh_params(dim: int = 4, n_tables: int = 3, n_proj: int = 4, w: float = 0.5, seed: int = 1):
    """Projection matrix alpha [dim, n_tables*n_proj] ~ N(0,1) and offsets beta [n_tables*n_proj] ~ U(0,w).
    Column c = table * n_proj + projection. Same draw calls as the reference's E2LSH constructor
    (``torch.normal(0, 1, (n_heads, dim, n_hashes))`` then a uniform in [0, r))."""
    gen = torch.Generator().manual_seed(seed)
    alpha = torch.normal(0.0, 1.0, (1, dim, n_tables * n_proj), generator=gen)[0].contiguous()
    beta = (torch.rand(1, n_tables * n_proj, generator=gen) * w)[0].contiguous()
    return alpha, beta


def gdr_inputs(B: int, T: int, H: int, K: int, V: int, dtype=torch.bfloat16, seed: int = 0, g_scale=1.0):
    """q, k ~ N(0,1) L2-normalised over the head dimension; v ~ N(0,1); beta = sigmoid(N(0,1));
    g = -g_scale * softplus(N(0,1)) (log-decay). q/k/v in ``dtype``; g, beta in fp32."""
    gen = torch.Generator().manual_seed(seed)
    q = torch.nn.functional.normalize(torch.randn(B, T, H, K, generator=gen), dim=-1)
    k = torch.nn.functional.normalize(torch.randn(B, T, H, K, generator=gen), dim=-1)
    v = torch.randn(B, T, H, V, generator=gen)
    beta = torch.sigmoid(torch.randn(B, T, H, generator=gen))
    g = -g_scale * torch.nn.functional.softplus(torch.randn(B, T, H, generator=gen))
    return q.to(dtype), k.to(dtype), v.to(dtype), g.float(), beta.float()


def varlen_lengths(n_seq: int = 16, lo: int = 6000, hi: int = 60000, seed: int = 0):
    """Sequence lengths ~ U[lo, hi] and their cumulative offsets (int64 [n_seq+1])."""
    gen = torch.Generator().manual_seed(seed)
    lens = torch.randint(lo, hi + 1, (n_seq,), generator=gen)
    cu = torch.zeros(n_seq + 1, dtype=torch.int64)
    cu[1:] = torch.cumsum(lens, 0)
    return lens, cu
