"""GPU parity of the gate kernel, a gated-delta layer and the `lshgd`-style block against the float64 CPU oracle.

The GPU path keeps activations in bf16 between operators (fp32 inside them); the oracle keeps float64 throughout. The
bounds below are therefore rounding budgets, stated per test: one layer (projection GEMMs, convolutions, gated delta,
gated norm, output GEMM, each rounding to bf16) to max-abs 2e-2 of the output scale and mean-rel 1e-2; the 4-layer block
to max-abs 5e-2 of the output scale and mean-rel 1e-2. Measured: 7e-3 / 6e-3 for a layer, 1e-2 / 7e-3 for the block."""
import numpy as np
import pytest
import torch

from lampa_amd import block as lb
from lampa_amd import layer_ops as lo
from lampa_amd import synth
from oracle import block as ob

pytestmark = pytest.mark.gpu


def _params(module):
    out = {}
    for k, v in module.state_dict().items():
        if k.endswith("_bits"):
            out[k[:-5]] = v.cpu().view(torch.float32).double().numpy()
        else:
            out[k] = v.detach().double().cpu().numpy()
    return out


def _errors(got, want):
    got = got.detach().double().cpu().numpy()
    scale = np.abs(want).max()
    return np.abs(got - want).max() / scale, np.abs(got - want).mean() / np.abs(want).mean()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gates_against_oracle(device, dtype):
    gen = torch.Generator().manual_seed(0)
    proj = (torch.randn(2, 700, 48, generator=gen) * 6).to(dtype).to(device)
    a, b = proj[..., 32:40], proj[..., 40:48]                              # column slices, read in place
    A_log, dt = torch.randn(8, generator=gen), torch.randn(8, generator=gen)
    g, beta = lo.gdr_gates(a, b, A_log.double().to(device), dt.double().to(device), 2.0)  # converted copies inside
    wg, wb = ob.gates(a.double().cpu().numpy(), b.double().cpu().numpy(), A_log.double().numpy(), dt.double().numpy(), 2.0)
    assert g.dtype == torch.float32 and g.shape == (2, 700, 8)
    assert np.allclose(g.cpu().numpy(), wg, rtol=2e-6, atol=1e-7) and np.allclose(beta.cpu().numpy(), wb, rtol=2e-6, atol=1e-7)
    assert (g <= 0).all()


@pytest.mark.parametrize("T,cu", [(1000, None), (777, [0, 100, 100, 401, 777])])
def test_gated_delta_layer_against_oracle(device, T, cu):
    torch.manual_seed(3)
    layer = lb.GatedDeltaLayer(hidden_size=128, head_dim=64, num_heads=8).to(device).to(torch.bfloat16)
    x = torch.randn(1, T, 128, device=device).bfloat16()
    cu_t = None if cu is None else torch.tensor(cu, device=device)
    y, _ = layer(x, cu_seqlens=cu_t)
    want = ob.gated_delta_layer({"l." + k: v for k, v in _params(layer).items()}, "l.", x.double().cpu().numpy(), 8, 64,
                                cu_seqlens=cu)
    max_rel, mean_rel = _errors(y, want)
    print(f"layer T={T}: max-abs/scale {max_rel:.2e}, mean-rel {mean_rel:.2e}, scale {np.abs(want).max():.3f}")
    assert y.shape == (1, T, 128) and y.dtype == torch.bfloat16
    assert max_rel < 2e-2 and mean_rel < 1e-2


@pytest.mark.parametrize("n_hits", [5000, 60000])
def test_lshgd_block_against_oracle(device, n_hits):
    torch.manual_seed(2)                                                   # the benchmark's weight seed
    block = lb.LshgdBlock().to(device).to(torch.bfloat16)
    coords, feats, _ = synth.collider_event(n_hits, seed=0)
    out = block(feats.to(device), coords.to(device))
    want = ob.lshgd_block(_params(block), feats.numpy(), coords.numpy(), 4, 8, 64, 3, 4, 0.5)
    max_rel, mean_rel = _errors(out, want)
    print(f"block N={n_hits}: max-abs/scale {max_rel:.2e}, mean-rel {mean_rel:.2e}, scale {np.abs(want).max():.3f}")
    assert out.shape == (n_hits, 24) and out.dtype == torch.bfloat16
    assert max_rel < 5e-2 and mean_rel < 1e-2
    # the hash parameters survive the cast of the module to bf16 bit for bit (seed 1)
    gen = torch.Generator().manual_seed(1)
    assert torch.equal(block.lsh_alpha.cpu(), torch.normal(0.0, 1.0, (4, 12), generator=gen))
