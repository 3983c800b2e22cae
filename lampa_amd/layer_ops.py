"""The operators either side of the gated-delta forward in a layer: the depthwise causal short convolution and the
(gated) RMS norm, as gfx950 kernels behind the reference's names.

Mirrors ``causal_conv1d`` / ``ShortConvolution`` (``models/hattention/short_convolution.py:426-458,528-721``) and
``rms_norm_gated`` / ``rms_norm`` / ``FusedRMSNormGated`` / ``FusedRMSNormSwishGate`` / ``RMSNorm``
(``models/hattention/fused_norm.py:856-878,1003-1104,2094-2354``). Forward only; GPU tensors only (no CPU fallback).
"""
import weakref
from typing import Optional, Tuple

import torch
import torch.nn as nn

from . import _capi
from ._capi import check, ptr, require_cuda, stream_of

_DTYPES = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}
_ACT = {None: 0, "silu": 1, "swish": 1, "sigmoid": 2}


class _ForwardOnly(torch.autograd.Function):
    """Lets the operators take part in a graph that is never differentiated; backward raises."""

    @staticmethod
    def forward(ctx, fn, *tensors):
        return fn()

    @staticmethod
    def backward(ctx, *grads):
        raise NotImplementedError("lampa_amd implements the forward pass of this operator only")


def _code(dtype) -> int:
    if dtype not in _DTYPES:
        raise TypeError(f"lampa_amd: unsupported dtype {dtype} (bfloat16, float16 or float32)")
    return _DTYPES[dtype]


_F32_CACHE = {}


def _root(t: torch.Tensor) -> torch.Tensor:
    return t._base if t._base is not None else t


def _stamp(t: torch.Tensor):
    r = _root(t)
    return (id(r), tuple(t.shape), tuple(t.stride()), t.storage_offset())


def _fresh(entry, parts) -> bool:
    """A remembered copy is valid while every source object is alive, unmoved and unmodified in place."""
    return entry is not None and all(ref() is _root(p) and ver == _root(p)._version and addr == p.data_ptr()
                                     for (ref, ver, addr), p in zip(entry[0], parts))


def _remember(key, parts, value):
    if len(_F32_CACHE) > 512:
        _F32_CACHE.clear()
    _F32_CACHE[key] = ([(weakref.ref(_root(p)), _root(p)._version, p.data_ptr()) for p in parts], value)
    return value


def _f32(t: Optional[torch.Tensor], device) -> Optional[torch.Tensor]:
    """fp32 contiguous copy of a small parameter on ``device``. Copies are remembered per source tensor object and
    dropped when it is modified in place, moved or freed, so a layer does not convert its weights on every call
    (edits made through ``.data`` bypass the version counter and are not noticed)."""
    if t is None:
        return None
    if t.dtype == torch.float32 and t.is_contiguous() and t.device == torch.device(device):
        return t.detach()
    key = ("one", _stamp(t), str(device))
    entry = _F32_CACHE.get(key)
    if _fresh(entry, [t]):
        return entry[1]
    return _remember(key, [t], t.detach().to(device=device, dtype=torch.float32).contiguous())


def _cat_f32(parts, device) -> torch.Tensor:
    key = ("cat", tuple(_stamp(p) for p in parts), str(device))
    entry = _F32_CACHE.get(key)
    if _fresh(entry, parts):
        return entry[1]
    return _remember(key, parts,
                     torch.cat([p.detach().to(device=device, dtype=torch.float32) for p in parts]).contiguous())


# ----------------------------------------------------------------------------------------------- short convolution
@torch.no_grad()
def _conv_launch(x2: torch.Tensor, weight, bias, residual2, activation, cu_seqlens, t_len: int, parts: int = 1):
    """x2 [tokens, D] (last dim contiguous, any row stride) -> y [tokens, D] contiguous, or [parts, tokens, D / parts]
    when the columns are split over ``parts`` output tensors."""
    n, D = x2.shape
    W = weight.shape[-1]
    split = D // parts
    y = torch.empty((n, D) if parts == 1 else (parts, n, split), dtype=x2.dtype, device=x2.device)
    if n == 0:
        return y
    cu = None if cu_seqlens is None else cu_seqlens.to(device=x2.device, dtype=torch.int64).contiguous()
    check(_capi.lib().lampa_causal_conv1d_fwd(
        ptr(x2), x2.stride(0), n, D, W, ptr(weight), ptr(bias), ptr(residual2),
        0 if residual2 is None else residual2.stride(0), ptr(cu), 0 if cu is None else cu.numel() - 1, t_len,
        _ACT[activation], _code(x2.dtype), ptr(y), split, split if parts > 1 else 0, n * split, stream_of(x2)),
        "lampa_causal_conv1d_fwd")
    return y


def _rows(t: torch.Tensor) -> torch.Tensor:
    """[B, T, D] -> [B*T, D] view with a contiguous last dimension (copies only when it has to)."""
    B, T, D = t.shape
    if t.stride(-1) != 1 or (B > 1 and t.stride(0) != T * t.stride(1)) or t.stride(1) % 8 or t.data_ptr() % 16:
        t = t.contiguous()
    return t.as_strided((B * T, D), (t.stride(1), 1))


def causal_conv1d(x: torch.Tensor, weight: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
                  residual: Optional[torch.Tensor] = None, activation: Optional[str] = None,
                  cu_seqlens: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``short_convolution.py:426-458``: x [B, T, D], weight [D, W] (tap W-1 on the current token), bias [D],
    residual [B, T, D]; activation ``None`` / ``'silu'`` / ``'swish'``; with ``cu_seqlens`` B must be 1 and taps never
    cross a sequence start. Returns [B, T, D] in x's dtype (fp32 arithmetic)."""
    require_cuda(x, weight, bias, residual, cu_seqlens)
    if activation not in (None, "silu", "swish"):
        raise ValueError(f"Activation `{activation}` not supported yet.")
    if x.dim() != 3:
        raise ValueError("causal_conv1d: x must be [B, T, D]")
    B, T, D = x.shape
    if cu_seqlens is not None and B != 1:
        raise ValueError("causal_conv1d: batch size must be 1 when cu_seqlens is given")
    if weight is None:
        weight = torch.ones(D, 1, device=x.device)
    w32, b32 = _f32(weight.reshape(D, -1), x.device), _f32(bias, x.device)
    res2 = None if residual is None else _rows(residual.to(x.dtype))
    x2 = _rows(x)
    fn = lambda: _conv_launch(x2, w32, b32, res2, activation, cu_seqlens, max(T, 1)).view(B, T, D)  # noqa: E731
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (x, weight, bias, residual)):
        return _ForwardOnly.apply(fn, x, weight)
    return fn()


@torch.no_grad()
def causal_conv1d_split(x: torch.Tensor, weights, biases=None, activation: Optional[str] = None,
                        cu_seqlens: Optional[torch.Tensor] = None):
    """One launch for several convolutions of equal width over adjacent column blocks of x [B, T, n * D] (the q | k | v
    columns of a fused projection): weights = n tensors [D, W] (or [D, 1, W]), biases = None or n tensors [D].
    Returns n contiguous tensors [B, T, D]. Same arithmetic as ``causal_conv1d`` on each block."""
    require_cuda(x, cu_seqlens, *weights)
    B, T, Dall = x.shape
    n = len(weights)
    D = Dall // n
    if Dall != n * D or any(w.numel() != weights[0].numel() or w.shape[0] != D for w in weights):
        raise ValueError("causal_conv1d_split: the column blocks must have equal width")
    if cu_seqlens is not None and B != 1:
        raise ValueError("causal_conv1d_split: batch size must be 1 when cu_seqlens is given")
    w32 = _cat_f32([w.reshape(D, -1) for w in weights], x.device)
    b32 = None if biases is None or biases[0] is None else _cat_f32(list(biases), x.device)
    y = _conv_launch(_rows(x), w32, b32, None, activation, cu_seqlens, max(T, 1), parts=n)
    return tuple(y[i].view(B, T, D) for i in range(n))


PROJ_CONV_HIDDEN = 128  # contraction length the fused projection kernel is built for


@torch.no_grad()
def proj_conv(x: torch.Tensor, weight: torch.Tensor, conv_weights, conv_biases, conv_split: int, plain_cols: int,
              tokens_per_wg: int = 0):
    """Fused bias-free projections + short convolution (4 taps) + SiLU: x [B, T, 128] bf16, weight [n_cols, 128] bf16
    (the projection weights one after the other), conv_weights = tensors [conv_split, 4] (or [conv_split, 1, 4]) for
    the first len(conv_weights) * conv_split columns, conv_biases = None or matching tensors. Returns
    (conv outputs: tuple of [B, T, conv_split], plain [B, T, plain_cols], tail [B, T, rest]); the projection output
    itself is never written. Same arithmetic as ``F.linear`` in bf16 followed by ``causal_conv1d(..., 'silu')``."""
    require_cuda(x, weight, *conv_weights)
    B, T, K = x.shape
    n_cols = weight.shape[0]
    n_conv = len(conv_weights) * conv_split
    tail = n_cols - n_conv - plain_cols
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or K != PROJ_CONV_HIDDEN or weight.shape[1] != K:
        raise ValueError("proj_conv: bf16 x [B, T, 128] and weight [n_cols, 128] expected")
    if any(w.shape[0] != conv_split or w.shape[-1] != 4 for w in conv_weights) or tail < 0:
        raise ValueError("proj_conv: conv_weights must be [conv_split, 4] each and fit the columns of weight")
    x2 = _rows(x)
    weight = weight.detach().contiguous()
    cw = _cat_f32([w.reshape(conv_split, 4) for w in conv_weights], x.device)
    cb = None if conv_biases is None or conv_biases[0] is None else _cat_f32(list(conv_biases), x.device)
    n = B * T
    y_conv = torch.empty((len(conv_weights), n, conv_split), dtype=x.dtype, device=x.device)
    y_plain = torch.empty((n, plain_cols), dtype=x.dtype, device=x.device)
    y_tail = torch.empty((n, tail), dtype=x.dtype, device=x.device)
    check(_capi.lib().lampa_proj_conv_fwd(ptr(x2), x2.stride(0), n, max(T, 1), K, ptr(weight), n_cols, ptr(cw), ptr(cb), n_conv,
                                          conv_split, ptr(y_conv), plain_cols, ptr(y_plain) if plain_cols else None, tail,
                                          ptr(y_tail) if tail else None, tokens_per_wg, stream_of(x)), "lampa_proj_conv_fwd")
    return (tuple(y_conv[i].view(B, T, conv_split) for i in range(len(conv_weights))), y_plain.view(B, T, plain_cols),
            y_tail.view(B, T, tail))


def norm_proj_supported(o: torch.Tensor, n_out: int) -> bool:
    """Shapes the fused gated-norm + output-projection kernel is built for."""
    return o.dtype == torch.bfloat16 and o.dim() == 4 and o.shape[2] * o.shape[3] == 512 and o.shape[3] == 64 and n_out == 128


@torch.no_grad()
def norm_proj(o: torch.Tensor, g: torch.Tensor, norm_weight: Optional[torch.Tensor], weight: torch.Tensor,
              eps: float = 1e-5, tokens_per_wg: int = 0, residual: Optional[torch.Tensor] = None,
              next_norm_weight: Optional[torch.Tensor] = None, next_eps: float = 1e-5):
    """``o_proj(FusedRMSNormSwishGate(o, g))`` in one kernel: o, g [B, T, 8, 64] bf16 (g may be a view with a token
    stride), norm_weight [64] or None, weight [128, 512] bf16 -> [B, T, 128]. The normalised tensor is rounded to bf16
    as the two-step route stores it, but never written. With ``residual`` [B, T, 128] (bf16) the kernel also applies the
    residual add and the next pre-norm, ``RMSNorm(next_norm_weight, next_eps)(y, residual, prenorm=True)``, and returns
    (normalised [B, T, 128], residual + y [B, T, 128])."""
    require_cuda(o, g, norm_weight, weight)
    if not norm_proj_supported(o, weight.shape[0]) or weight.dtype != torch.bfloat16 or weight.shape[1] != 512:
        raise ValueError("norm_proj: bf16 o [B, T, 8, 64] and weight [128, 512] expected")
    B, T, H, D = o.shape
    o = o.contiguous()
    g = g.to(o.dtype)
    if not (g.stride(-1) == 1 and g.stride(-2) == D and g.stride(1) % 8 == 0 and g.data_ptr() % 16 == 0
            and (B == 1 or g.stride(0) == T * g.stride(1))):
        g = g.contiguous()
    w32 = _f32(norm_weight, o.device)
    weight = weight.detach().contiguous()
    y = torch.empty((B, T, weight.shape[0]), dtype=o.dtype, device=o.device)
    res_out, nw32 = None, None
    if residual is not None:
        require_cuda(residual, next_norm_weight)
        if residual.shape != y.shape or residual.dtype != o.dtype:
            raise ValueError("norm_proj: residual must be bf16 [B, T, 128]")
        residual = residual.contiguous()
        res_out = torch.empty_like(y)
        nw32 = _f32(next_norm_weight, o.device)
    check(_capi.lib().lampa_norm_proj_fwd(ptr(o), ptr(g), g.stride(1), ptr(w32), ptr(weight), B * T, H, D, weight.shape[0],
                                          float(eps), ptr(y), ptr(residual), ptr(nw32), float(next_eps), ptr(res_out),
                                          tokens_per_wg, stream_of(o)), "lampa_norm_proj_fwd")
    return y if residual is None else (y, res_out)


class ShortConvolution(nn.Conv1d):
    """``short_convolution.py:528-721``: depthwise causal convolution over the time axis of a [B, T, D] tensor with
    an optional SiLU, a cache of the last W inputs per sequence ([N, D, W]) and a one-token ``step``."""

    def __init__(self, hidden_size: int, kernel_size: int, bias: bool = False, activation: Optional[str] = 'silu',
                 use_fast_conv1d: Optional[bool] = True, device=None, dtype=None, **kwargs):
        super().__init__(in_channels=hidden_size, out_channels=hidden_size, kernel_size=kernel_size, groups=hidden_size,
                         bias=bias, padding=kernel_size - 1, device=device, dtype=dtype)
        self.hidden_size = hidden_size
        self.activation = None
        if kernel_size % 2 != 0:
            raise ValueError("Kernel size must be the power of 2")
        if activation is not None:
            assert activation in ['silu', 'swish'], f"Activation `{activation}` not supported yet."
            self.activation = activation
        self.use_fast_conv1d = False  # one implementation here: the HIP kernel

    def forward(self, x: torch.Tensor, residual: Optional[torch.Tensor] = None, mask: Optional[torch.Tensor] = None,
                cache: Optional[torch.Tensor] = None, output_final_state: bool = False,
                cu_seqlens: Optional[torch.LongTensor] = None, **kwargs) -> Tuple[torch.Tensor, torch.Tensor]:
        B, T, D, W = *x.shape, self.kernel_size[0]
        N = B if cu_seqlens is None else len(cu_seqlens) - 1
        if mask is not None:
            if cu_seqlens is not None:
                raise ValueError("`mask` and `cu_seqlens` cannot be provided at the same time")
            x = x.mul_(mask.unsqueeze(-1))
        if output_final_state and cache is None:
            cache = x.new_zeros(N, D, W)
        if cache is not None and B * T == N:
            return self.step(x, residual, cache, cu_seqlens)
        if cache is not None:
            with torch.no_grad():
                if cu_seqlens is not None:
                    cu = cu_seqlens.to(x.device).long()
                    idx = cu[1:, None] - W + torch.arange(W, device=x.device)[None]          # [N, W]
                    ok = idx >= torch.maximum(cu[:-1], cu[1:] - W)[:, None]
                    rows = x[0][idx.clamp(min=0)] * ok[..., None].to(x.dtype)                # [N, W, D]
                    cache.copy_(rows.transpose(1, 2))
                else:
                    cache[:, :, -min(W, T):].copy_(x[..., -min(W, T):, :].transpose(1, 2))
        y = causal_conv1d(x=x, weight=self.weight.reshape(D, W), bias=self.bias, residual=residual,
                          activation=self.activation, cu_seqlens=cu_seqlens)
        return y, cache

    def step(self, x: torch.Tensor, residual: Optional[torch.Tensor], cache: torch.Tensor,
             cu_seqlens: Optional[torch.LongTensor] = None):
        """One token per sequence: the cache is rolled in place, then the convolution runs over its W columns."""
        shape = x.shape
        D, W = self.hidden_size, self.kernel_size[0]
        xt = x.reshape(-1, D)
        with torch.no_grad():
            cache.copy_(cache.roll(shifts=-1, dims=-1))
            cache[:, :, -1] = xt
            window = cache.transpose(1, 2).contiguous()                                       # [N, W, D]
        y = causal_conv1d(x=window, weight=self.weight.reshape(D, W), bias=self.bias, activation=self.activation)
        y = y[:, -1].reshape(shape)
        if residual is not None:
            y = y + residual
        return y, cache

    @property
    def state_size(self) -> int:
        return self.hidden_size * self.kernel_size


# ------------------------------------------------------------------------------------------------------ RMS norm
@torch.no_grad()
def _norm_launch(x2, g2, weight, bias, residual2, residual_dtype, eps, activation, g_group=0, g_group_stride=0):
    rows, D = x2.shape
    y = torch.empty_like(x2)
    want_res_out = residual2 is not None or (residual_dtype is not None and residual_dtype != x2.dtype)
    res_out = torch.empty((rows, D), dtype=residual_dtype, device=x2.device) if want_res_out else None
    if rows:
        check(_capi.lib().lampa_rms_norm_fwd(
            ptr(x2), ptr(g2), ptr(weight), ptr(bias), ptr(residual2), ptr(res_out), ptr(y), None, rows, D, float(eps),
            _ACT[activation] if g2 is not None else 0, _code(x2.dtype),
            _code(residual_dtype) if want_res_out else _code(x2.dtype), g_group, g_group_stride, stream_of(x2)),
            "lampa_rms_norm_fwd")
    return y, (res_out if res_out is not None else x2)


def _rms_norm_any(x, g, weight, bias, activation, residual, eps, prenorm, residual_in_fp32):
    require_cuda(x, g, weight, bias, residual)
    shape = x.shape
    D = shape[-1]
    x2 = x.reshape(-1, D).contiguous()
    g2, g_group, g_group_stride = None, 0, 0
    if g is not None:
        g = g.to(x.dtype)
        # [..., T, H, D] view of the g_proj columns of a wider projection output: read in place
        if (g.dim() >= 3 and not g.is_contiguous() and g.stride(-1) == 1 and g.stride(-2) == D and g.stride(-3) % 8 == 0
                and g.data_ptr() % 16 == 0 and g.stride(-3) >= g.shape[-2] * D
                and all(g.stride(i) == g.stride(i + 1) * g.shape[i + 1] for i in range(g.dim() - 3))):
            g2, g_group, g_group_stride = g, g.shape[-2], g.stride(-3)
        else:
            g2 = g.reshape(-1, D).contiguous()
    if residual is not None:
        assert residual.shape == shape
    res2 = None if residual is None else residual.reshape(-1, D).contiguous()
    residual_dtype = res2.dtype if res2 is not None else (torch.float32 if residual_in_fp32 else None)
    w32, b32 = _f32(weight, x.device), _f32(bias, x.device)

    def fn():
        y, res_out = _norm_launch(x2, g2, w32, b32, res2, residual_dtype, eps, activation, g_group, g_group_stride)
        return (y.reshape(shape), res_out.reshape(shape)) if prenorm else y.reshape(shape)

    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (x, g, weight, bias, residual)):
        return _ForwardOnly.apply(fn, x)
    return fn()


def rms_norm_gated(x: torch.Tensor, g: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, activation: str = 'swish',
                   residual: Optional[torch.Tensor] = None, prenorm: bool = False, residual_in_fp32: bool = False,
                   eps: float = 1e-6):
    """``fused_norm.py:856-878``: y = rmsnorm(x + residual) * weight + bias, times ``g * sigmoid(g)`` ('swish' /
    'silu') or ``sigmoid(g)`` ('sigmoid'); the norm runs over the last dimension. ``prenorm`` also returns x + residual."""
    if activation not in ('swish', 'silu', 'sigmoid'):
        raise ValueError(f"Unsupported activation: {activation}")
    return _rms_norm_any(x, g, weight, bias, activation, residual, eps, prenorm, residual_in_fp32)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, residual: torch.Tensor = None, eps: float = 1e-5,
             prenorm: bool = False, residual_in_fp32: bool = False):
    """``fused_norm.py:2094-2112``: y = rmsnorm(x + residual) * weight + bias; ``prenorm`` also returns x + residual."""
    return _rms_norm_any(x, None, weight, bias, None, residual, eps, prenorm, residual_in_fp32)


class FusedRMSNormGated(nn.Module):
    """``fused_norm.py:1003-1064``."""

    def __init__(self, hidden_size: int, elementwise_affine: bool = True, eps: float = 1e-5, activation: str = 'swish',
                 device=None, dtype=None):
        super().__init__()
        self.hidden_size = hidden_size
        self.elementwise_affine = elementwise_affine
        self.eps = eps
        self.activation = activation
        if self.activation not in ['swish', 'silu', 'sigmoid']:
            raise ValueError(f"Unsupported activation: {self.activation}")
        if elementwise_affine:
            self.weight = nn.Parameter(torch.ones(hidden_size, device=device, dtype=dtype))
        else:
            self.register_parameter("weight", None)
        self.register_parameter("bias", None)

    def forward(self, x: torch.Tensor, g: torch.Tensor, residual: Optional[torch.Tensor] = None, prenorm: bool = False,
                residual_in_fp32: bool = False) -> torch.Tensor:
        return rms_norm_gated(x, g, self.weight, self.bias, self.activation, residual=residual, eps=self.eps,
                              prenorm=prenorm, residual_in_fp32=residual_in_fp32)


class FusedRMSNormSwishGate(FusedRMSNormGated):
    """``fused_norm.py:1088-1104``."""

    def __init__(self, hidden_size: int, elementwise_affine: bool = True, eps: float = 1e-5, device=None, dtype=None):
        super().__init__(hidden_size=hidden_size, elementwise_affine=elementwise_affine, eps=eps, device=device,
                         dtype=dtype)


class RMSNorm(nn.Module):
    """``fused_norm.py:2307-2354``."""

    def __init__(self, hidden_size: int, elementwise_affine: bool = True, bias: bool = False, eps: float = 1e-5):
        super().__init__()
        self.hidden_size = hidden_size
        self.elementwise_affine = elementwise_affine
        self.eps = eps
        self.register_parameter("weight", None)
        self.register_parameter("bias", None)
        if elementwise_affine:
            self.weight = nn.Parameter(torch.ones(hidden_size))
            if bias:
                self.bias = nn.Parameter(torch.zeros(hidden_size))

    def forward(self, x, residual=None, prenorm=False, residual_in_fp32=False):
        return rms_norm(x, self.weight, self.bias, residual=residual, eps=self.eps, prenorm=prenorm,
                        residual_in_fp32=residual_in_fp32)


# ----------------------------------------------------------------------------------------- decay and write gates
@torch.no_grad()
def gdr_gates(a: torch.Tensor, b: torch.Tensor, A_log: torch.Tensor, dt_bias: torch.Tensor, beta_scale: float = 1.0):
    """``modeling_gated_deltaproduct.py:541-547,568-570``: g = -exp(A_log) * softplus(a + dt_bias) and
    beta = sigmoid(b) * beta_scale, both fp32 [..., H]. a, b [..., H] may be column slices of a wider projection."""
    require_cuda(a, b, A_log, dt_bias)
    H = a.shape[-1]
    assert b.shape == a.shape and a.dtype == b.dtype

    def rows(t):
        if t.dim() >= 2 and t.stride(-1) == 1 and all(t.stride(i) == t.stride(i + 1) * t.shape[i + 1]
                                                      for i in range(t.dim() - 2)):
            return t, t.stride(-2) if t.dim() >= 2 else H
        t = t.contiguous()
        return t, H

    a2, a_stride = rows(a)
    b2, b_stride = rows(b)
    n = a.numel() // H
    g = torch.empty(a.shape, dtype=torch.float32, device=a.device)
    beta = torch.empty_like(g)
    A32, dt32 = _f32(A_log, a.device), _f32(dt_bias, a.device)  # named: they must outlive the launch call
    if n:
        check(_capi.lib().lampa_gdr_gates_fwd(ptr(a2), a_stride, ptr(b2), b_stride, ptr(A32), ptr(dt32), n, H,
                                              float(beta_scale), _code(a.dtype), ptr(g), ptr(beta), stream_of(a)),
              "lampa_gdr_gates_fwd")
    return g, beta
