"""Writes the small regression fixtures of this directory from the CPU oracle.

The reference ships no golden vectors for this path and its kernels cannot run here, so these files are NOT reference
outputs: they freeze what the pinned oracle computes on fixed seeded inputs, so that a later change to the oracle, to the
synthetic generators or to the HIP kernels shows up as a diff against committed numbers. Run from the repository root:

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from lampa_amd import synth  # noqa: E402  (seeded input generators only; no GPU code runs here)
from oracle import gated_delta as og  # noqa: E402
from oracle import hgdn as oh  # noqa: E402
from oracle import lsh as ol  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def lsh_fixture():
    coords, feats, _ = synth.collider_event(256, seed=7)
    alpha, beta = synth.lsh_params(4, 3, 4, 0.5, 1)
    out = ol.bucket_sort(coords.numpy(), alpha.numpy(), beta.numpy(), 0.5, 3, 4, feats.numpy(), n_valid=250)
    np.savez_compressed(os.path.join(HERE, "lsh_event256.npz"), coords=coords.numpy(), feats=feats.numpy(),
                        alpha=alpha.numpy(), beta=beta.numpy(), ids=out["ids"], keys=out["keys"], meta=out["meta"],
                        perm=out["perm"], sorted_feats=out["feats"].astype(np.float32))


def gdr_fixture():
    q, k, v, g, beta = synth.gdr_inputs(1, 96, 2, 64, 64, torch.bfloat16, seed=5, g_scale=0.05)
    h0 = 0.5 * torch.randn(1, 2, 64, 64, generator=torch.Generator().manual_seed(6))
    o, s = og.recurrent_c(q, k, v, g, beta, initial_state=h0, l2=og.L2_CHUNK, dtype=torch.float64)
    np.savez_compressed(os.path.join(HERE, "gdr_t96_h2_d64.npz"), q=q.float().numpy(), k=k.float().numpy(),
                        v=v.float().numpy(), g=g.numpy(), beta=beta.numpy(), h0=h0.numpy(), o=o.numpy(),
                        final_state=s.numpy())


def hgdn_fixture():
    # three chunks, two heads: levels 0..8 (the 7 inside a chunk and two chunk-index bits); lambda as it enters the
    # operator (the operator divides it by scale = 1/8)
    q, k, v, g, beta = synth.gdr_inputs(1, 192, 2, 64, 64, torch.bfloat16, seed=8, g_scale=0.2)
    lam = (torch.rand(1, 192, 2, 9, generator=torch.Generator().manual_seed(9)) + 0.25).bfloat16()
    o = oh.recurrent_c(q, k, v, g, beta, lam / 0.125, scale=0.125)
    np.savez_compressed(os.path.join(HERE, "hgdn_t192_h2_d64.npz"), q=q.float().numpy(), k=k.float().numpy(),
                        v=v.float().numpy(), g=g.numpy(), beta=beta.numpy(), lam=lam.float().numpy(), o=o.numpy())


if __name__ == "__main__":
    lsh_fixture()
    gdr_fixture()
    hgdn_fixture()
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
