"""A gated-delta layer and the `lshgd`-style block built from this package's operators.

``GatedDeltaLayer`` follows ``GatedDeltaProduct`` with one householder step (``models/hattention/
modeling_gated_deltaproduct.py:317-625``): q/k/v projections -> short convolution + SiLU -> l2-normalised chunkwise
gated-delta forward with decay g = -exp(A_log) softplus(a + dt_bias) and write strength beta = sigmoid(b) -> RMS norm
gated by swish(g_proj(x)) -> output projection. ``LshgdBlock`` is the benchmark block: input linear, LSH bucket sort of
the hits, pre-norm residual layers (the fused add + norm of ``GatedDeltaProductBlock.forward``, ``:1029-1056``), unsort
and an embedding head. The projections are plain library GEMMs (one fused GEMM per layer for q|k|v|g|b|a); everything
else runs in this package's HIP kernels. Forward only.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import lsh
from .gated_delta import chunk_gated_delta_rule
from .layer_ops import (PROJ_CONV_HIDDEN, FusedRMSNormSwishGate, RMSNorm, ShortConvolution, causal_conv1d,
                        causal_conv1d_split, gdr_gates, norm_proj, norm_proj_supported, proj_conv)


class GatedDeltaLayer(nn.Module):
    def __init__(self, hidden_size: int = 128, head_dim: int = 64, num_heads: int = 8, expand_v: float = 1,
                 conv_size: int = 4, norm_eps: float = 1e-6, allow_neg_eigval: bool = False):
        super().__init__()
        self.hidden_size, self.head_dim, self.num_heads = hidden_size, head_dim, num_heads
        self.key_dim = num_heads * head_dim
        self.value_dim = int(self.key_dim * expand_v)
        self.head_v_dim = int(head_dim * expand_v)
        self.allow_neg_eigval = allow_neg_eigval
        self.q_proj = nn.Linear(hidden_size, self.key_dim, bias=False)
        self.k_proj = nn.Linear(hidden_size, self.key_dim, bias=False)
        self.v_proj = nn.Linear(hidden_size, self.value_dim, bias=False)
        self.g_proj = nn.Linear(hidden_size, self.value_dim, bias=False)
        self.b_proj = nn.Linear(hidden_size, num_heads, bias=False)
        self.a_proj = nn.Linear(hidden_size, num_heads, bias=False)
        self.q_conv1d = ShortConvolution(self.key_dim, conv_size, activation="silu")
        self.k_conv1d = ShortConvolution(self.key_dim, conv_size, activation="silu")
        self.v_conv1d = ShortConvolution(self.value_dim, conv_size, activation="silu")
        # decay parameters as in modeling_gated_deltaproduct.py:420-437
        A = torch.empty(num_heads, dtype=torch.float32).uniform_(0, 16)
        self.A_log = nn.Parameter(torch.log(A))
        dt = torch.exp(torch.rand(num_heads) * (math.log(0.1) - math.log(0.001)) + math.log(0.001)).clamp(min=1e-4)
        self.dt_bias = nn.Parameter(dt + torch.log(-torch.expm1(-dt)))
        self.o_norm = FusedRMSNormSwishGate(self.head_v_dim, eps=norm_eps)
        self.o_proj = nn.Linear(self.value_dim, hidden_size, bias=False)
        self._fused = None

    def _fused_weight(self):
        parts = (self.q_proj.weight, self.k_proj.weight, self.v_proj.weight, self.g_proj.weight, self.b_proj.weight,
                 self.a_proj.weight)
        key = tuple((p.data_ptr(), p._version, p.dtype) for p in parts)
        if self._fused is None or self._fused[0] != key:
            self._fused = (key, torch.cat([p.detach() for p in parts], dim=0).contiguous())
        return self._fused[1]

    @torch.no_grad()
    def forward(self, hidden_states: torch.Tensor, cu_seqlens=None, initial_state=None, output_final_state=False,
                residual=None, next_norm=None):
        """hidden_states [B, T, hidden] -> (o [B, T, hidden], final_state or None). With ``residual`` and ``next_norm``
        (an ``RMSNorm``) the layer also applies the residual add and that norm and returns
        ((next_norm(o + residual), o + residual), final_state): the pre-norm wiring of a stack of layers, fused into
        the output projection kernel when the shapes allow it."""
        B, T, _ = hidden_states.shape
        H, dk, dv, kd, vd = self.num_heads, self.head_dim, self.head_v_dim, self.key_dim, self.value_dim
        convs = (self.q_conv1d, self.k_conv1d, self.v_conv1d)
        fused = (cu_seqlens is None and hidden_states.dtype == torch.bfloat16 and self.hidden_size == PROJ_CONV_HIDDEN
                 and kd == vd and kd % 256 == 0 and (2 * H) % 8 == 0)
        if fused:  # projections, convolutions and SiLU in one kernel: the projection output never reaches memory
            (q, k, v), xg, xba = proj_conv(hidden_states, self._fused_weight(), [c.weight for c in convs],
                                           [c.bias for c in convs], kd, vd)
            xb, xa = xba[..., :H], xba[..., H:]
        else:
            proj = F.linear(hidden_states, self._fused_weight())                 # [B, T, 2 kd + 2 vd + 2 H]
            cols = [0, kd, 2 * kd, 2 * kd + vd, 2 * kd + 2 * vd, 2 * kd + 2 * vd + H, 2 * kd + 2 * vd + 2 * H]
            xq, xk, xv, xg, xb, xa = (proj[..., cols[i]:cols[i + 1]] for i in range(6))
            if kd == vd:                                                         # one launch over the q | k | v columns
                q, k, v = causal_conv1d_split(proj[..., :cols[3]], [c.weight for c in convs], [c.bias for c in convs],
                                              "silu", cu_seqlens)
            else:
                q, k, v = (causal_conv1d(t, c.weight.reshape(t.shape[-1], -1), c.bias, None, "silu", cu_seqlens)
                           for t, c in zip((xq, xk, xv), convs))
        g, beta = gdr_gates(xa, xb, self.A_log, self.dt_bias, 2.0 if self.allow_neg_eigval else 1.0)
        o, state = chunk_gated_delta_rule(q.view(B, T, H, dk), k.view(B, T, H, dk), v.view(B, T, H, dv), g, beta,
                                          initial_state=initial_state, output_final_state=output_final_state,
                                          cu_seqlens=cu_seqlens, use_qk_l2norm_in_kernel=True)
        gate = xg.unflatten(-1, (H, dv))
        if norm_proj_supported(o, self.hidden_size) and self.o_proj.weight.dtype == torch.bfloat16:  # norm + gate + GEMM
            if residual is not None and residual.dtype == torch.bfloat16 and next_norm.bias is None:
                return norm_proj(o, gate, self.o_norm.weight, self.o_proj.weight, self.o_norm.eps, residual=residual,
                                 next_norm_weight=next_norm.weight, next_eps=next_norm.eps), state
            out = norm_proj(o, gate, self.o_norm.weight, self.o_proj.weight, self.o_norm.eps)
        else:
            out = self.o_proj(self.o_norm(o, gate).reshape(B, T, vd))
        return (out if residual is None else next_norm(out, residual, True)), state


class LshgdBlock(nn.Module):
    """Input linear -> LSH bucket sort of the hits -> ``n_layers`` pre-norm residual gated-delta layers -> final norm ->
    unsort -> embedding head. Parameters are created under the caller's seed with torch's default Linear / Conv1d
    initialisation (Kaiming-uniform)."""

    def __init__(self, in_dim: int = 24, hidden: int = 128, n_layers: int = 4, num_heads: int = 8, head_dim: int = 64,
                 out_dim: int = 24, coord_dim: int = 4, n_tables: int = 3, n_proj: int = 4, bucket_width: float = 0.5,
                 lsh_seed: int = 1):
        super().__init__()
        self.input = nn.Linear(in_dim, hidden)
        self.norms = nn.ModuleList([RMSNorm(hidden, eps=1e-6) for _ in range(n_layers)])
        self.layers = nn.ModuleList([GatedDeltaLayer(hidden, head_dim, num_heads) for _ in range(n_layers)])
        self.norm_f = RMSNorm(hidden, eps=1e-6)
        self.head = nn.Linear(hidden, out_dim)
        self.n_tables, self.n_proj, self.bucket_width = n_tables, n_proj, bucket_width
        gen = torch.Generator().manual_seed(lsh_seed)
        alpha = torch.normal(0.0, 1.0, (coord_dim, n_tables * n_proj), generator=gen)
        beta = torch.rand(n_tables * n_proj, generator=gen) * bucket_width
        # kept as bit patterns so that module.to(bfloat16) leaves the float32 hash parameters alone
        self.register_buffer("lsh_alpha_bits", alpha.view(torch.int32))
        self.register_buffer("lsh_beta_bits", beta.view(torch.int32))
        self._flags_host = None  # pinned copy of the LSH stage's flag fields (one per table), made on first use

    @property
    def lsh_alpha(self) -> torch.Tensor:
        return self.lsh_alpha_bits.view(torch.float32)

    @property
    def lsh_beta(self) -> torch.Tensor:
        return self.lsh_beta_bits.view(torch.float32)

    @torch.no_grad()
    def order(self, coords: torch.Tensor, check: bool = True):
        """Sequence order of the hits: the stable bucket-sort permutation of the first hash table (int32 [N]).
        ``check=True`` reads the flag field of the stage at once (one host synchronisation): when a workgroup of the
        one-launch kernel gave up a wait (``lsh.META_GAVE_UP``) the stage runs again as separate kernels, which wait for
        nothing; a key that does not fit 32 bits raises. ``check=False`` returns ``(perm, pending)`` instead and leaves
        the flags to ``_flags_of(pending)``: they are copied to pinned host memory behind the kernel, so that the caller
        can queue its other launches first and look at them without draining the stream."""
        args = (coords.float(), self.lsh_alpha, self.lsh_beta, self.bucket_width, self.n_tables, self.n_proj)
        out = lsh.lsh_bucket_sort(*args, return_ids=False)
        if not check:
            if self._flags_host is None:
                self._flags_host = torch.empty(self.n_tables, dtype=torch.int32, pin_memory=True)
            self._flags_host.copy_(out["meta"][..., -1], non_blocking=True)
            done = torch.cuda.Event()
            done.record()
            return out["perm"][0], done
        flags = lsh.decode_meta_flags(out["meta"])
        if bool(flags["gave_up"].any()):
            return self._order_with_separate_kernels(args)
        if bool(flags["key_overflow"][0]):
            raise lsh.LampaError("LshgdBlock: the bucket key of the first hash table does not fit 32 bits; the "
                                 "sequence order would be meaningless")
        return out["perm"][0]

    def _order_with_separate_kernels(self, args):
        lsh.one_launch_config(enabled=False)
        try:
            return lsh.lsh_bucket_sort(*args, return_ids=False, strict=True)["perm"][0]
        finally:
            lsh.one_launch_config(enabled=True)

    def _flags_of(self, done) -> int:
        """The flag fields of the last ``order(check=False)`` call, OR-ed over the tables (waits for that kernel only)."""
        done.synchronize()
        flags = 0
        for f in self._flags_host.tolist():
            flags |= f
        return flags

    @torch.no_grad()
    def forward(self, feats: torch.Tensor, coords: torch.Tensor, perm: torch.Tensor = None) -> torch.Tensor:
        """feats [N, in_dim], coords [N, coord_dim] -> [N, out_dim] in the parameters' dtype, in the input hit order.
        The LSH stage's flag field is looked at once per event, after every launch of the block has been queued: a
        one-launch kernel that gave up a wait (its permutation is then all -1) makes the block run again with the order
        from the separate kernels; a key overflow raises."""
        dtype = self.input.weight.dtype
        pending = None
        if perm is None:
            perm, pending = self.order(coords, check=False)
        x = self.input(feats.to(dtype))
        x = lsh.gather_rows(x[None], perm[None])                                 # [1, N, hidden], LSH order
        h, residual = self.norms[0](x, None, True)                               # residual = x, h = norm(x)
        for i, layer in enumerate(self.layers):                                  # residual <- out + residual; h = next norm
            next_norm = self.norms[i + 1] if i + 1 < len(self.layers) else self.norm_f
            (h, residual), _ = layer(h, residual=residual, next_norm=next_norm)
        h = lsh.scatter_rows(h, perm[None])[0]                                   # back to the input order
        out = self.head(h)
        if pending is not None:
            flags = self._flags_of(pending)
            if flags & lsh.META_GAVE_UP:
                args = (coords.float(), self.lsh_alpha, self.lsh_beta, self.bucket_width, self.n_tables, self.n_proj)
                return self.forward(feats, coords, perm=self._order_with_separate_kernels(args))
            if self._flags_host[0].item() & lsh.META_KEY_OVERFLOW:
                raise lsh.LampaError("LshgdBlock: the bucket key of the first hash table does not fit 32 bits; the "
                                     "sequence order would be meaningless")
        return out
