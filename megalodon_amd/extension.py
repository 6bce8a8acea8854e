"""Python face of the C ABI with the reference's operator signatures.

Each function here has the name, argument order, returned tuple and error
behaviour of one function of the reference's pybind module
``megalodon_extension.ops`` (megalodon/csrc/megalodon_extension.cc:14-24) and
forwards to the matching ``mega_*`` entry point of ``libmegalodon_hip.so``.
Outputs are allocated here with ``torch.empty`` on the inputs' device (the
reference allocates them inside the C++ op); kernels run on the current
stream; nothing synchronises.  Non-CUDA tensors raise ``RuntimeError``: there
is no CPU path in this package.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib


def _require_cuda(*tensors) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("megalodon_amd ops need GPU (HIP) tensors; there is no CPU fallback")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError("all tensors must be on the same device")
    return dev


def _as_c64(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.dtype != torch.complex64:
        raise RuntimeError(f"{name} must be complex64 (got {t.dtype})")
    return t.contiguous()


# --------------------------------------------------------------------------
# ema_parameters (reference: csrc/ops/ema_parameters.cc:195-290)
# --------------------------------------------------------------------------
def ema_parameters_fwd(
    p: torch.Tensor,
    log_q: torch.Tensor,
    gamma: torch.Tensor,
    h: Optional[torch.Tensor],
    L: int,
) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """(w, b, v) = ema_parameters_fwd(p, log_q, gamma, h, L); weight path only.

    p (D,N[,1]) float32, log_q/gamma complex64 -> w (D, L) float32.  With
    ``h`` given the reference also returns the bias of the carried state
    (ema_parameters.cc:56-77); that branch is not part of this library yet.
    """
    dev = _require_cuda(p, log_q, gamma, h)
    if h is not None:
        raise NotImplementedError("ema_parameters with a carried state (h) is not implemented")
    if p.dtype != torch.float32:
        raise RuntimeError(f"p must be float32 (got {p.dtype})")
    D, N = p.shape[0], p.shape[1]
    p_c = p.contiguous()
    lq = _as_c64(log_q, "log_q")
    gm = _as_c64(gamma, "gamma")
    w = torch.empty((D, L), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_ema_weight_fwd", _lib.ptr(p_c), _lib.ptr(lq), _lib.ptr(gm),
                  _lib.i64(D), _lib.i64(N), _lib.i64(L), _lib.ptr(w), _lib.stream_ptr(dev))
    return w, None, None


def ema_parameters_bwd(
    w_grad: torch.Tensor,
    b_grad: Optional[torch.Tensor],
    p: torch.Tensor,
    log_q: torch.Tensor,
    gamma: torch.Tensor,
    h: Optional[torch.Tensor],
    v: Optional[torch.Tensor],
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """(dp, dq, dgamma, dh); gradients w.r.t. q (not log q), PyTorch conjugate
    convention (ema_parameters.cc:80-98)."""
    dev = _require_cuda(w_grad, p, log_q, gamma, h, b_grad)
    if h is not None or b_grad is not None:
        raise NotImplementedError("ema_parameters with a carried state (h) is not implemented")
    if p.dtype != torch.float32 or w_grad.dtype != torch.float32:
        raise RuntimeError("p and w_grad must be float32")
    D, N = p.shape[0], p.shape[1]
    L = w_grad.shape[-1]
    dw = w_grad.contiguous()
    p_c = p.contiguous()
    lq = _as_c64(log_q, "log_q")
    gm = _as_c64(gamma, "gamma")
    dp = torch.empty_like(p_c)
    dq = torch.empty_like(lq)
    dg = torch.empty_like(gm)
    with torch.cuda.device(dev):
        _lib.call("mega_ema_weight_bwd", _lib.ptr(dw), _lib.ptr(p_c), _lib.ptr(lq), _lib.ptr(gm),
                  _lib.i64(D), _lib.i64(N), _lib.i64(L), _lib.ptr(dp), _lib.ptr(dq), _lib.ptr(dg),
                  _lib.stream_ptr(dev))
    return dp, dq, dg, None


# --------------------------------------------------------------------------
# fftconv (reference: csrc/ops/fftconv.cc:22-33, fused_ops/fftconv.py:30-106)
# --------------------------------------------------------------------------
def fftconv_max_length() -> int:
    return int(_lib.load().mega_fftconv_max_length())


def fftconv_fwd(x: torch.Tensor, k: torch.Tensor) -> torch.Tensor:
    """y = causal_conv(x, k).  x (B, D, L) float32/bfloat16/float16, k (D, L).

    Differs from the reference's ``fftconv_fwd(x, k_f) -> (y, x_f)`` in taking
    the time-domain kernel and returning no saved spectrum: backward recomputes
    it (1 GiB of ``x_f`` is not kept alive between forward and backward)."""
    dev = _require_cuda(x, k)
    if x.dim() != 3 or k.dim() != 2 or k.shape[0] != x.shape[1] or k.shape[1] != x.shape[2]:
        raise RuntimeError(f"fftconv: x {tuple(x.shape)} and k {tuple(k.shape)} do not match (B,D,L)/(D,L)")
    B, D, L = x.shape
    xc = x.contiguous()
    kc = k.contiguous().float()
    y = torch.empty_like(xc)
    with torch.cuda.device(dev):
        _lib.call("mega_fftconv_fwd", _lib.ptr(xc), _lib.i32(_lib.dtype_code(x.dtype)), _lib.ptr(kc),
                  _lib.i64(B), _lib.i64(D), _lib.i64(L), _lib.ptr(y), _lib.stream_ptr(dev))
    return y


def fftconv_bwd(y_grad: torch.Tensor, x: torch.Tensor, k: torch.Tensor,
                k_dtype: torch.dtype) -> Tuple[torch.Tensor, torch.Tensor]:
    """(dx, dk) with dk of dtype ``k_dtype`` (fftconv.py:53-75)."""
    dev = _require_cuda(y_grad, x, k)
    B, D, L = x.shape
    if y_grad.shape != x.shape or y_grad.dtype != x.dtype:
        raise RuntimeError("fftconv_bwd: y_grad must match x in shape and dtype")
    dy = y_grad.contiguous()
    xc = x.contiguous()
    kc = k.contiguous().float()
    dx = torch.empty_like(xc)
    dk = torch.empty((D, L), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_fftconv_bwd", _lib.ptr(dy), _lib.ptr(xc), _lib.i32(_lib.dtype_code(x.dtype)),
                  _lib.ptr(kc), _lib.i64(B), _lib.i64(D), _lib.i64(L), _lib.ptr(dx), _lib.ptr(dk),
                  _lib.stream_ptr(dev))
    return dx, dk.to(k_dtype)


def fftconv_residual_fwd(x: torch.Tensor, k: torch.Tensor, omega: torch.Tensor) -> torch.Tensor:
    """y = causal_conv(x, k) + omega[d] * x in one kernel: the convolution and the
    skip term of MultiHeadComplexEMA.forward
    (complex_exponential_moving_average.py:136-146).  omega (D,) or (D, 1)."""
    dev = _require_cuda(x, k, omega)
    if x.dim() != 3 or k.dim() != 2 or k.shape[0] != x.shape[1] or k.shape[1] != x.shape[2]:
        raise RuntimeError(f"fftconv: x {tuple(x.shape)} and k {tuple(k.shape)} do not match (B,D,L)/(D,L)")
    if omega.numel() != x.shape[1]:
        raise RuntimeError(f"fftconv: omega has {omega.numel()} elements for D={x.shape[1]}")
    B, D, L = x.shape
    xc = x.contiguous()
    kc = k.contiguous().float()
    wc = omega.reshape(-1).contiguous().float()
    y = torch.empty_like(xc)
    with torch.cuda.device(dev):
        _lib.call("mega_fftconv_residual_fwd", _lib.ptr(xc), _lib.i32(_lib.dtype_code(x.dtype)),
                  _lib.ptr(kc), _lib.ptr(wc), _lib.i64(B), _lib.i64(D), _lib.i64(L), _lib.ptr(y),
                  _lib.stream_ptr(dev))
    return y


def fftconv_residual_bwd(y_grad: torch.Tensor, x: torch.Tensor, k: torch.Tensor,
                         omega: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dx, dk, domega) of ``fftconv_residual_fwd``; dk and domega are float32.
    domega is the lag-0 column of dk: sum_b sum_t dy[b,d,t] x[b,d,t]."""
    dev = _require_cuda(y_grad, x, k, omega)
    B, D, L = x.shape
    if y_grad.shape != x.shape or y_grad.dtype != x.dtype:
        raise RuntimeError("fftconv_bwd: y_grad must match x in shape and dtype")
    dy = y_grad.contiguous()
    xc = x.contiguous()
    kc = k.contiguous().float()
    wc = omega.reshape(-1).contiguous().float()
    dx = torch.empty_like(xc)
    dk = torch.empty((D, L), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_fftconv_residual_bwd", _lib.ptr(dy), _lib.ptr(xc),
                  _lib.i32(_lib.dtype_code(x.dtype)), _lib.ptr(kc), _lib.ptr(wc), _lib.i64(B),
                  _lib.i64(D), _lib.i64(L), _lib.ptr(dx), _lib.ptr(dk), _lib.stream_ptr(dev))
    return dx, dk, dk[:, 0].clone()


# --------------------------------------------------------------------------
# group_timestep_norm (reference: csrc/ops/timestep_norm.cc:621-705)
# --------------------------------------------------------------------------
def _tsn_workspace(B, L, D, G, backward, dev):
    fn = _lib.load().mega_group_timestep_norm_workspace_bytes
    fn.restype = _lib.ctypes.c_int64
    nbytes = int(fn(_lib.i64(B), _lib.i64(L), _lib.i64(D), _lib.i64(G), _lib.i32(1 if backward else 0)))
    return torch.empty(nbytes, dtype=torch.uint8, device=dev)


def _mask_bytes(padding_mask):
    if padding_mask is None:
        return None
    if padding_mask.dtype != torch.bool:
        raise RuntimeError("padding_mask must be a bool tensor")
    return padding_mask.contiguous().view(torch.uint8)


def group_timestep_norm_fwd(
    x: torch.Tensor,
    prev_count: torch.Tensor,
    prev_mean: torch.Tensor,
    prev_var: torch.Tensor,
    gamma: torch.Tensor,
    beta: torch.Tensor,
    padding_mask: Optional[torch.Tensor],
    num_groups: int,
    eps: float,
):
    """(y, count, mean, var, cummean, cumrstd); tensors other than count /
    mask / the float32 statistics must share x's dtype, as in the reference
    (timestep_norm_kernel.cu:1270-1273)."""
    dev = _require_cuda(x, prev_count, prev_mean, prev_var, gamma, beta, padding_mask)
    if x.dim() != 3:
        raise RuntimeError("x must be (B, L, D)")
    B, L, D = x.shape
    for name, t in (("prev_mean", prev_mean), ("prev_var", prev_var), ("gamma", gamma), ("beta", beta)):
        if t.dtype != x.dtype:
            raise RuntimeError(f"{name} must have x's dtype {x.dtype} (got {t.dtype})")
    if prev_count.dtype != torch.int64:
        raise RuntimeError("prev_count must be int64")
    G = int(num_groups)
    xc = x.contiguous()
    y = torch.empty_like(xc)
    count = torch.empty_like(prev_count, memory_format=torch.contiguous_format)
    mean = torch.empty((B, G), dtype=x.dtype, device=dev)
    var = torch.empty((B, G), dtype=x.dtype, device=dev)
    cummean = torch.empty((B, L, G), dtype=torch.float32, device=dev)
    cumrstd = torch.empty((B, L, G), dtype=torch.float32, device=dev)
    mask = _mask_bytes(padding_mask)
    ws = _tsn_workspace(B, L, D, G, False, dev)
    with torch.cuda.device(dev):
        _lib.call("mega_group_timestep_norm_fwd", _lib.ptr(xc), _lib.i32(_lib.dtype_code(x.dtype)),
                  _lib.ptr(prev_count.contiguous()), _lib.ptr(prev_mean.contiguous()),
                  _lib.ptr(prev_var.contiguous()), _lib.ptr(gamma.contiguous()), _lib.ptr(beta.contiguous()),
                  _lib.ptr(mask), _lib.i64(B), _lib.i64(L), _lib.i64(D), _lib.i64(G), _lib.f64(eps),
                  _lib.ptr(y), _lib.ptr(count), _lib.ptr(mean), _lib.ptr(var), _lib.ptr(cummean),
                  _lib.ptr(cumrstd), _lib.ptr(ws), _lib.stream_ptr(dev))
    return y, count, mean, var, cummean, cumrstd


def group_timestep_norm_bwd(
    y_grad: torch.Tensor,
    mean_grad: torch.Tensor,
    var_grad: torch.Tensor,
    x: torch.Tensor,
    prev_mean: torch.Tensor,
    count: torch.Tensor,
    cummean: torch.Tensor,
    cumrstd: torch.Tensor,
    gamma: torch.Tensor,
    padding_mask: Optional[torch.Tensor],
    num_groups: int,
):
    """(dx, dprev_mean, dprev_var, dgamma, dbeta)."""
    dev = _require_cuda(y_grad, mean_grad, var_grad, x, prev_mean, count, cummean, cumrstd, gamma, padding_mask)
    B, L, D = x.shape
    G = int(num_groups)
    for name, t in (("y_grad", y_grad), ("mean_grad", mean_grad), ("var_grad", var_grad),
                    ("prev_mean", prev_mean), ("gamma", gamma)):
        if t.dtype != x.dtype:
            raise RuntimeError(f"{name} must have x's dtype {x.dtype} (got {t.dtype})")
    xc, dy = x.contiguous(), y_grad.contiguous()
    dx = torch.empty_like(xc)
    dpm = torch.empty((B, G), dtype=x.dtype, device=dev)
    dpv = torch.empty((B, G), dtype=x.dtype, device=dev)
    dg = torch.empty((D,), dtype=x.dtype, device=dev)
    db = torch.empty((D,), dtype=x.dtype, device=dev)
    mask = _mask_bytes(padding_mask)
    ws = _tsn_workspace(B, L, D, G, True, dev)
    with torch.cuda.device(dev):
        _lib.call("mega_group_timestep_norm_bwd", _lib.ptr(dy), _lib.ptr(mean_grad.contiguous()),
                  _lib.ptr(var_grad.contiguous()), _lib.ptr(xc), _lib.i32(_lib.dtype_code(x.dtype)),
                  _lib.ptr(prev_mean.contiguous()), _lib.ptr(count.contiguous()),
                  _lib.ptr(cummean.contiguous()), _lib.ptr(cumrstd.contiguous()), _lib.ptr(gamma.contiguous()),
                  _lib.ptr(mask), _lib.i64(B), _lib.i64(L), _lib.i64(D), _lib.i64(G), _lib.ptr(dx),
                  _lib.ptr(dpm), _lib.ptr(dpv), _lib.ptr(dg), _lib.ptr(db), _lib.ptr(ws),
                  _lib.stream_ptr(dev))
    return dx, dpm, dpv, dg, db


# --------------------------------------------------------------------------
# attention (reference: csrc/ops/attention.cc:28-29, attention_kernel.cu:261-303)
# --------------------------------------------------------------------------
def _attn_workspace(B, L1, L2, NH, H1, H2, backward, dev):
    fn = _lib.load().mega_attention_workspace_bytes
    fn.restype = _lib.ctypes.c_int64
    nbytes = int(fn(_lib.i64(B), _lib.i64(L1), _lib.i64(L2), _lib.i64(NH), _lib.i64(H1), _lib.i64(H2),
                    _lib.i32(1 if backward else 0)))
    return torch.empty(nbytes, dtype=torch.uint8, device=dev)


def _attn_dims(q, k, v):
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise RuntimeError("q, k, v must be (B, L, N, H)")
    B, L1, NH, H1 = q.shape
    L2, H2 = k.shape[1], v.shape[3]
    if k.shape != (B, L2, NH, H1) or v.shape != (B, L2, NH, H2):
        raise RuntimeError(f"attention: inconsistent shapes q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)}")
    if not (q.dtype == k.dtype == v.dtype):
        raise RuntimeError("q, k, v must share one dtype")
    return B, L1, L2, NH, H1, H2


def attention_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, dropout: float,
                  use_causal_mask: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """(y, w): y (B, L1, N, H2), w = softmax probabilities (B, N, L1, L2)."""
    dev = _require_cuda(q, k, v)
    if dropout != 0.0:
        raise NotImplementedError("DropKey dropout is not implemented (dropout must be 0)")
    B, L1, L2, NH, H1, H2 = _attn_dims(q, k, v)
    qc, kc, vc = q.contiguous(), k.contiguous(), v.contiguous()
    y = torch.empty((B, L1, NH, H2), dtype=v.dtype, device=dev)
    w = torch.empty((B, NH, L1, L2), dtype=v.dtype, device=dev)
    ws = _attn_workspace(B, L1, L2, NH, H1, H2, False, dev)
    with torch.cuda.device(dev):
        _lib.call("mega_attention_fwd", _lib.ptr(qc), _lib.ptr(kc), _lib.ptr(vc),
                  _lib.i32(_lib.dtype_code(q.dtype)), _lib.i64(B), _lib.i64(L1), _lib.i64(L2), _lib.i64(NH),
                  _lib.i64(H1), _lib.i64(H2), _lib.f64(scale), _lib.i32(1 if use_causal_mask else 0),
                  _lib.ptr(y), _lib.ptr(w), _lib.ptr(ws), _lib.stream_ptr(dev))
    return y, w


def attention_bwd(y_grad: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, w: torch.Tensor,
                  scale: float, use_causal_mask: bool) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dq, dk, dv)."""
    dev = _require_cuda(y_grad, q, k, v, w)
    B, L1, L2, NH, H1, H2 = _attn_dims(q, k, v)
    if w.shape != (B, NH, L1, L2) or y_grad.shape != (B, L1, NH, H2):
        raise RuntimeError("attention_bwd: w / y_grad shapes do not match q, k, v")
    qc, kc, vc, dy, wc = q.contiguous(), k.contiguous(), v.contiguous(), y_grad.contiguous(), w.contiguous()
    dq, dk, dv = torch.empty_like(qc), torch.empty_like(kc), torch.empty_like(vc)
    ws = _attn_workspace(B, L1, L2, NH, H1, H2, True, dev)
    with torch.cuda.device(dev):
        _lib.call("mega_attention_bwd", _lib.ptr(dy), _lib.ptr(qc), _lib.ptr(kc), _lib.ptr(vc), _lib.ptr(wc),
                  _lib.i32(_lib.dtype_code(q.dtype)), _lib.i64(B), _lib.i64(L1), _lib.i64(L2), _lib.i64(NH),
                  _lib.i64(H1), _lib.i64(H2), _lib.f64(scale), _lib.i32(1 if use_causal_mask else 0),
                  _lib.ptr(dq), _lib.ptr(dk), _lib.ptr(dv), _lib.ptr(ws), _lib.stream_ptr(dev))
    return dq, dk, dv
