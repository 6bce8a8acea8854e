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


def _as_c64(t: torch.Tensor, name: str, wide: bool = False) -> torch.Tensor:
    """Contiguous complex64 tensor -- complex128 for the double-precision flavour (`wide`)."""
    want = torch.complex128 if wide else torch.complex64
    if t.dtype != want:
        raise RuntimeError(f"{name} must be {str(want)[6:]} (got {t.dtype})")
    return t.contiguous()


def _real_of(wide: bool) -> torch.dtype:
    return torch.float64 if wide else torch.float32


def _p_is_wide(p: torch.Tensor, who: str = "p") -> bool:
    """p float32 (complex64 companions) or float64 (complex128 companions), as the reference
    dispatches (ema_parameters_kernel.cu:1227)."""
    if p.dtype not in (torch.float32, torch.float64):
        raise RuntimeError(f"{who} must be float32 or float64 (got {p.dtype})")
    return p.dtype == torch.float64


# --------------------------------------------------------------------------
# ema_parameters (reference: csrc/ops/ema_parameters.cc:195-290)
# --------------------------------------------------------------------------
def _weight_rows(coef: torch.Tensor, log_q_rows: torch.Tensor, L: int) -> torch.Tensor:
    """rows[r, j] = sum_n Re(coef[r, n] q[r, n]^j), j < L: the weight kernel with
    one complex coefficient per (row, mode) (p = 1, gamma = coef)."""
    R, N = coef.shape
    dev = coef.device
    wide = coef.dtype == torch.complex128
    ones = torch.ones((R, N), dtype=_real_of(wide), device=dev)
    out = torch.empty((R, L), dtype=_real_of(wide), device=dev)
    cf, lq = coef.contiguous(), log_q_rows.contiguous()
    with torch.cuda.device(dev):
        _lib.call("mega_ema_weight_fwd_f64" if wide else "mega_ema_weight_fwd", _lib.ptr(ones), _lib.ptr(lq), _lib.ptr(cf), _lib.i64(R),
                  _lib.i64(N), _lib.i64(L), _lib.ptr(out), _lib.stream_ptr(dev))
    return out


def _row_moments(rows: torch.Tensor, log_q_rows: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """(S2, S1)[r, n] = (sum_j rows[r, j] q^j, sum_j j rows[r, j] q^(j-1)): the
    weight-backward kernel with p = gamma = 1, whose dgamma = conj(S2) and
    dq = conj(S1) (ema_parameters.cc:80-98)."""
    R, L = rows.shape
    N = log_q_rows.shape[1]
    dev = rows.device
    wide = log_q_rows.dtype == torch.complex128
    ones = torch.ones((R, N), dtype=_real_of(wide), device=dev)
    onec = torch.ones((R, N), dtype=log_q_rows.dtype, device=dev)
    dp = torch.empty((R, N), dtype=_real_of(wide), device=dev)
    dq = torch.empty((R, N), dtype=log_q_rows.dtype, device=dev)
    dg = torch.empty((R, N), dtype=log_q_rows.dtype, device=dev)
    rw, lq = rows.to(_real_of(wide)).contiguous(), log_q_rows.contiguous()
    with torch.cuda.device(dev):
        _lib.call("mega_ema_weight_bwd_f64" if wide else "mega_ema_weight_bwd", _lib.ptr(rw), _lib.ptr(ones), _lib.ptr(lq), _lib.ptr(onec),
                  _lib.i64(R), _lib.i64(N), _lib.i64(L), _lib.ptr(dp), _lib.ptr(dq), _lib.ptr(dg),
                  _lib.stream_ptr(dev))
    return dg.conj().resolve_conj(), dq.conj().resolve_conj()


def _qpow(log_q: torch.Tensor, k: int) -> torch.Tensor:
    """q^k in log_q's precision, evaluated in complex128 (k * arg q loses bits in float32)."""
    return torch.exp(log_q.to(torch.complex128) * float(k)).to(log_q.dtype)


def ema_parameters_fwd(
    p: torch.Tensor,
    log_q: torch.Tensor,
    gamma: torch.Tensor,
    h: Optional[torch.Tensor],
    L: int,
) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """(w, b, v) = ema_parameters_fwd(p, log_q, gamma, h, L).

    p (D,N[,1]) float32, log_q/gamma complex64 -> w (D, L) float32 (float64 /
    complex128 -> float64: the double-precision flavour).  With the
    carried state ``h`` (B, D, N) complex64 also the bias
    ``b[b,d,j] = sum_n Re(q^(j+1) gamma h[b,d,n])`` (B, D, L)
    (ema_parameters.cc:56-77): the weight kernel run on the B*D rows with the
    coefficient q*gamma*h.  ``v`` (the reference's Vandermonde scratch for B > 8)
    is never needed and stays ``None``.
    """
    dev = _require_cuda(p, log_q, gamma, h)
    wide = _p_is_wide(p)
    D, N = p.shape[0], p.shape[1]
    p_c = p.contiguous()
    lq = _as_c64(log_q, "log_q", wide)
    gm = _as_c64(gamma, "gamma", wide)
    w = torch.empty((D, L), dtype=p.dtype, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_ema_weight_fwd_f64" if wide else "mega_ema_weight_fwd", _lib.ptr(p_c), _lib.ptr(lq),
                  _lib.ptr(gm), _lib.i64(D), _lib.i64(N), _lib.i64(L), _lib.ptr(w), _lib.stream_ptr(dev))
    if h is None:
        return w, None, None
    hc = _as_c64(h, "h", wide)
    if hc.dim() != 3 or hc.shape[1] != D or hc.shape[2] != N:
        raise RuntimeError(f"h must be (B, {D}, {N}) (got {tuple(hc.shape)})")
    B = hc.shape[0]
    lq2, gm2 = lq.reshape(D, N), gm.reshape(D, N)
    coef = (torch.exp(lq2) * gm2).unsqueeze(0) * hc
    lq_rows = lq2.unsqueeze(0).expand(B, D, N).reshape(B * D, N)
    b = _weight_rows(coef.reshape(B * D, N), lq_rows, L).view(B, D, L)
    return w, b, None


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
    convention (ema_parameters.cc:80-98; bias part :100-117,158-188)."""
    dev = _require_cuda(w_grad, p, log_q, gamma, h, b_grad)
    wide = _p_is_wide(p)
    if w_grad.dtype != p.dtype:
        raise RuntimeError(f"p and w_grad must share float32 or float64 (got {p.dtype}, {w_grad.dtype})")
    D, N = p.shape[0], p.shape[1]
    L = w_grad.shape[-1]
    dw = w_grad.contiguous()
    p_c = p.contiguous()
    lq = _as_c64(log_q, "log_q", wide)
    gm = _as_c64(gamma, "gamma", wide)
    dp = torch.empty_like(p_c)
    dq = torch.empty_like(lq)
    dg = torch.empty_like(gm)
    with torch.cuda.device(dev):
        _lib.call("mega_ema_weight_bwd_f64" if wide else "mega_ema_weight_bwd", _lib.ptr(dw), _lib.ptr(p_c), _lib.ptr(lq), _lib.ptr(gm),
                  _lib.i64(D), _lib.i64(N), _lib.i64(L), _lib.ptr(dp), _lib.ptr(dq), _lib.ptr(dg),
                  _lib.stream_ptr(dev))
    if b_grad is None:
        return dp, dq, dg, (torch.zeros_like(h) if h is not None else None)
    if h is None:
        raise RuntimeError("ema_parameters_bwd: a bias gradient needs the carried state h")
    hc = _as_c64(h, "h", wide)
    B = hc.shape[0]
    lq2, gm2 = lq.reshape(D, N), gm.reshape(D, N)
    lq_rows = lq2.unsqueeze(0).expand(B, D, N).reshape(B * D, N)
    s2, s1 = _row_moments(b_grad.reshape(B * D, L), lq_rows)
    s2, s1 = s2.view(B, D, N), s1.view(B, D, N)
    q = torch.exp(lq2)
    sum2 = q * s2               # sum_i db_i q^(i+1)
    sum1 = q * s1 + s2          # sum_i (i+1) db_i q^i
    dq = dq + torch.conj(sum1 * gm2 * hc).sum(dim=0).reshape(dq.shape)
    dg = dg + torch.conj(sum2 * hc).sum(dim=0).reshape(dg.shape)
    dh = torch.conj(sum2 * gm2)
    return dp, dq, dg, dh


# --------------------------------------------------------------------------
# CEMA coefficients (reference: modules/complex_exponential_moving_average.py:100-117)
# --------------------------------------------------------------------------
def _coeff_shapes(alpha, delta, theta, gamma):
    D, N = alpha.shape[0], alpha.shape[1]
    if alpha.numel() != D * N or delta.shape != alpha.shape or theta.numel() != D or gamma.numel() != 2 * D * N:
        raise RuntimeError("cema_coeffs: expected alpha, delta (D, N, 1), theta (D, 1, 1), gamma (D, N, 2)")
    for name, t in (("alpha", alpha), ("delta", delta), ("theta", theta), ("gamma", gamma)):
        if t.dtype != torch.float32:
            raise RuntimeError(f"cema_coeffs: {name} must be float32 (got {t.dtype})")
    return D, N


def cema_coeffs_fwd(alpha: torch.Tensor, delta: torch.Tensor, theta: torch.Tensor, gamma: torch.Tensor):
    """(p (D, N, 1) float32, log_q (D, N, 1) complex64, gamma_hat (D, N) complex64) in
    one launch: ``_calc_coeffs`` followed by ``q.log()``."""
    dev = _require_cuda(alpha, delta, theta, gamma)
    D, N = _coeff_shapes(alpha, delta, theta, gamma)
    a, d, t, g = alpha.contiguous(), delta.contiguous(), theta.contiguous(), gamma.contiguous()
    p = torch.empty((D, N, 1), dtype=torch.float32, device=dev)
    log_q = torch.empty((D, N, 1), dtype=torch.complex64, device=dev)
    gamma_hat = torch.empty((D, N), dtype=torch.complex64, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_cema_coeffs_fwd", _lib.ptr(a), _lib.ptr(d), _lib.ptr(t), _lib.ptr(g), _lib.i64(D),
                  _lib.i64(N), _lib.ptr(p), _lib.ptr(log_q), _lib.ptr(gamma_hat), _lib.stream_ptr(dev))
    return p, log_q, gamma_hat


def cema_coeffs_bwd(dp: torch.Tensor, dq: torch.Tensor, dgamma_hat: torch.Tensor, alpha: torch.Tensor,
                    delta: torch.Tensor, theta: torch.Tensor):
    """(dalpha, ddelta, dtheta, dgamma) from the gradients ``ema_parameters_bwd``
    returns (dp real, dq / dgamma_hat complex, PyTorch's convention)."""
    dev = _require_cuda(dp, dq, dgamma_hat, alpha, delta, theta)
    D, N = alpha.shape[0], alpha.shape[1]
    a, d, t = alpha.contiguous(), delta.contiguous(), theta.contiguous()
    dpc = dp.contiguous().float()
    dqc, dgc = _as_c64(dq, "dq"), _as_c64(dgamma_hat, "dgamma_hat")
    dalpha, ddelta, dtheta = torch.empty_like(a), torch.empty_like(d), torch.empty_like(t)
    dgamma = torch.empty((D, N, 2), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_cema_coeffs_bwd", _lib.ptr(dpc), _lib.ptr(dqc), _lib.ptr(dgc), _lib.ptr(a), _lib.ptr(d),
                  _lib.ptr(t), _lib.i64(D), _lib.i64(N), _lib.ptr(dalpha), _lib.ptr(ddelta), _lib.ptr(dtheta),
                  _lib.ptr(dgamma), _lib.stream_ptr(dev))
    return dalpha, ddelta, dtheta, dgamma


# --------------------------------------------------------------------------
# ema_hidden (reference: csrc/ops/ema_hidden.cc:16-159, fused_ops/ema_hidden.py)
# --------------------------------------------------------------------------
def ema_hidden_fwd(
    x: torch.Tensor,
    p: torch.Tensor,
    log_q: torch.Tensor,
    h: Optional[torch.Tensor],
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Last EMA state ``y[b,d,n] = p sum_j q^(L-1-j) x[b,d,j] (+ q^L h)``
    (ema_hidden.cc:16-62) and the saved moments ``v`` for backward.

    The time-reversed rows go through the weight-backward kernel, whose two sums
    over a row are exactly ``sum_i q^i x'[i]`` and ``sum_i i q^(i-1) x'[i]``;
    ``v`` stacks them (2, B, D, N) in place of the reference's Vandermonde tensor.
    x (B, D, L) any float dtype; p (D,N[,1]) float32; log_q complex64."""
    dev = _require_cuda(x, p, log_q, h)
    wide = _p_is_wide(p)
    B, D, L = x.shape
    N = p.shape[1]
    lq2 = _as_c64(log_q, "log_q", wide).reshape(D, N)
    lq_rows = lq2.unsqueeze(0).expand(B, D, N).reshape(B * D, N)
    s2, s1 = _row_moments(x.flip(-1).reshape(B * D, L), lq_rows)
    s2, s1 = s2.view(B, D, N), s1.view(B, D, N)
    y = p.reshape(D, N) * s2
    if h is not None:
        y = y + _qpow(lq2, L) * _as_c64(h, "h", wide)
    return y, torch.stack([s2, s1])


def ema_hidden_bwd(
    y_grad: torch.Tensor,
    x: torch.Tensor,
    p: torch.Tensor,
    log_q: torch.Tensor,
    h: Optional[torch.Tensor],
    v: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """(dx, dp, dq, dh) of ``ema_hidden_fwd`` (ema_hidden.cc:64-159)."""
    dev = _require_cuda(y_grad, x, p, log_q, h, v)
    B, D, L = x.shape
    N = p.shape[1]
    wide = _p_is_wide(p)
    lq2 = _as_c64(log_q, "log_q", wide).reshape(D, N)
    lq_rows = lq2.unsqueeze(0).expand(B, D, N).reshape(B * D, N)
    p2 = p.reshape(D, N)
    dyc = torch.conj(_as_c64(y_grad, "y_grad", wide)).resolve_conj()
    s2, s1 = v[0], v[1]
    # dx[j] = sum_n Re(conj(dy) p q^(L-1-j)): the weight kernel, then reversed in time
    dx = _weight_rows((dyc * p2).reshape(B * D, N), lq_rows, L).view(B, D, L).flip(-1).to(x.dtype)
    dp = (dyc * s2).real.sum(dim=0).reshape(p.shape)
    dq_sum = (dyc * p2 * s1).sum(dim=0)
    dh = None
    if h is not None:
        hc = _as_c64(h, "h", wide)
        dq_sum = dq_sum + (dyc * hc).sum(dim=0) * _qpow(lq2, L - 1) * float(L)
        dh = torch.conj(dyc * _qpow(lq2, L))
    dq = torch.conj(dq_sum).reshape(log_q.shape)
    return dx, dp, dq, dh


# --------------------------------------------------------------------------
# fftconv (reference: csrc/ops/fftconv.cc:22-33, fused_ops/fftconv.py:30-106)
# --------------------------------------------------------------------------
def fftconv_max_length() -> int:
    return int(_lib.load().mega_fftconv_max_length())


# Rows longer than one kernel launch takes are cut into nb blocks of S samples
# (zero padded at the end).  With head(a, c) = the first S outputs of the
# linear convolution of two blocks (what one launch computes) and tail(a, c) =
# its outputs S .. 2S-1,
#   y_b = sum_{i+j=b} head(x_i, k_j) + sum_{i+j=b-1} tail(x_i, k_j),
# and the tail is a head of the reversed blocks:
#   tail(a, c)[t] = head(flip a, flip c)[S-2-t]  (t <= S-2),  tail[S-1] = 0.
# All blocks x_i that meet one kernel block k_j go through one launch, stacked
# along the batch axis; the backward pass sends the gradient of every term
# through the backward launch of the same pair (which also sums dk over the
# stack).  Sums over terms are float32.  The reference takes rows of any
# length through torch.fft (fused_ops/fftconv.py:84,103).
def _long_blocks(L: int) -> Tuple[int, int]:
    nb = -(-L // fftconv_max_length())
    S = -(-L // nb)
    return nb, (S + 7) // 8 * 8


def _cut(t: torch.Tensor, nb: int, S: int) -> torch.Tensor:
    """(..., L) -> (nb, ..., S), zero padded."""
    L = t.shape[-1]
    if nb * S != L:
        t = torch.nn.functional.pad(t, (0, nb * S - L))
    return t.reshape(*t.shape[:-1], nb, S).movedim(-2, 0).contiguous()


def _fftconv_long_fwd(x: torch.Tensor, k: torch.Tensor, blocks=None, head=None) -> torch.Tensor:
    """`blocks` = (nb, S) and `head` = the one-launch operator; the defaults are
    the library's limits and `fftconv_fwd` (tests pass others)."""
    B, D, L = x.shape
    nb, S = blocks or _long_blocks(L)
    head = head or fftconv_fwd
    xb, kb = _cut(x, nb, S), _cut(k.float(), nb, S)
    xr, kr = xb.flip(-1), kb.flip(-1)
    y = torch.zeros((B, D, nb, S), dtype=torch.float32, device=x.device)  # the row, block by block
    for j in range(nb):
        n = nb - j
        y[:, :, j:] += head(xb[:n].reshape(n * B, D, S), kb[j]).view(n, B, D, S).permute(1, 2, 0, 3)
        n = nb - 1 - j
        if n > 0:
            h = head(xr[:n].reshape(n * B, D, S), kr[j]).view(n, B, D, S).permute(1, 2, 0, 3)
            y[:, :, j + 1:, :S - 1] += h[..., :S - 1].flip(-1)  # tail[t] = h[S-2-t]
    return y.view(B, D, nb * S)[..., :L].to(x.dtype)


def _fftconv_long_bwd(y_grad: torch.Tensor, x: torch.Tensor, k: torch.Tensor, blocks=None,
                      head_bwd=None) -> Tuple[torch.Tensor, torch.Tensor]:
    B, D, L = x.shape
    nb, S = blocks or _long_blocks(L)
    head_bwd = head_bwd or (lambda g, a, c: fftconv_bwd(g, a, c, torch.float32))
    xb, kb, gb = _cut(x, nb, S), _cut(k.float(), nb, S), _cut(y_grad, nb, S)
    xr, kr = xb.flip(-1), kb.flip(-1)
    dx = torch.zeros((B, D, nb, S), dtype=torch.float32, device=x.device)
    dk = torch.zeros((D, nb, S), dtype=torch.float32, device=x.device)
    for j in range(nb):
        n = nb - j
        gx, gk = head_bwd(gb[j:].reshape(n * B, D, S), xb[:n].reshape(n * B, D, S), kb[j])
        dx[:, :, :n] += gx.view(n, B, D, S).permute(1, 2, 0, 3)
        dk[:, j] += gk
        n = nb - 1 - j
        if n > 0:
            # gradient of h from the gradient of the tail: the same index reversal
            gh = torch.zeros((n, B, D, S), dtype=gb.dtype, device=x.device)
            gh[..., :S - 1] = gb[j + 1:, ..., :S - 1].flip(-1)
            gx, gk = head_bwd(gh.reshape(n * B, D, S), xr[:n].reshape(n * B, D, S), kr[j])
            dx[:, :, :n] += gx.view(n, B, D, S).permute(1, 2, 0, 3).flip(-1)
            dk[:, j] += gk.flip(-1)
    return dx.view(B, D, nb * S)[..., :L].to(x.dtype), dk.view(D, nb * S)[..., :L].contiguous()


def _causal_conv_f64(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """out[r, t] = sum_{s <= t} a[r % Ra, s] b[r, t - s] for float64 rows a (Ra, L), b (R, L): the
    double-precision flavour's convolution, the triangular sum itself (no transform)."""
    Ra, L = a.shape
    R = b.shape[0]
    ac, bc = a.contiguous(), b.contiguous()
    out = torch.empty_like(bc)
    with torch.cuda.device(b.device):
        _lib.call("mega_causal_conv_f64", _lib.ptr(ac), _lib.ptr(bc), _lib.i64(Ra), _lib.i64(R), _lib.i64(L),
                  _lib.ptr(out), _lib.stream_ptr(b.device))
    return out


def _fftconv_f64_fwd(x: torch.Tensor, k: torch.Tensor) -> torch.Tensor:
    B, D, L = x.shape
    return _causal_conv_f64(k.double(), x.reshape(B * D, L)).view(B, D, L)


def _fftconv_f64_bwd(y_grad: torch.Tensor, x: torch.Tensor, k: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """dx[t] = sum_s k[s] dy[t + s] and dk[j] = sum_b sum_t dy[t] x[t - j] are causal
    convolutions of the time-reversed gradient: flip(conv(k, flip dy)), sum_b flip(conv(x, flip dy))."""
    B, D, L = x.shape
    dyr = y_grad.flip(-1).reshape(B * D, L)
    dx = _causal_conv_f64(k.double(), dyr).flip(-1).view(B, D, L)
    dk = _causal_conv_f64(x.reshape(B * D, L), dyr).flip(-1).view(B, D, L).sum(dim=0)
    return dx, dk


def fftconv_fwd(x: torch.Tensor, k: torch.Tensor) -> torch.Tensor:
    """y = causal_conv(x, k).  x (B, D, L) float32/bfloat16/float16, k (D, L).

    Differs from the reference's ``fftconv_fwd(x, k_f) -> (y, x_f)`` in taking
    the time-domain kernel and returning no saved spectrum: backward recomputes
    it (1 GiB of ``x_f`` is not kept alive between forward and backward).

    With a complex ``k`` the call is the reference's own: ``fftconv_fwd(x, k_f)
    -> (y, x_f)`` (see ``_fftconv_fwd_spectral``)."""
    if k.is_complex():
        return _fftconv_fwd_spectral(x, k)
    dev = _require_cuda(x, k)
    if x.dim() != 3 or k.dim() != 2 or k.shape[0] != x.shape[1] or k.shape[1] != x.shape[2]:
        raise RuntimeError(f"fftconv: x {tuple(x.shape)} and k {tuple(k.shape)} do not match (B,D,L)/(D,L)")
    B, D, L = x.shape
    if x.dtype == torch.float64:
        return _fftconv_f64_fwd(x, k)
    if L > fftconv_max_length():
        return _fftconv_long_fwd(x, k)
    xc = x.contiguous()
    kc = k.contiguous().float()
    y = torch.empty_like(xc)
    with torch.cuda.device(dev):
        _lib.call("mega_fftconv_fwd", _lib.ptr(xc), _lib.i32(_lib.dtype_code(x.dtype)), _lib.ptr(kc),
                  _lib.i64(B), _lib.i64(D), _lib.i64(L), _lib.ptr(y), _lib.stream_ptr(dev))
    return y


def fftconv_bwd(y_grad: torch.Tensor, x: torch.Tensor, k: torch.Tensor,
                k_dtype: torch.dtype) -> Tuple[torch.Tensor, torch.Tensor]:
    """(dx, dk) with dk of dtype ``k_dtype`` (fftconv.py:53-75).  With complex
    ``x`` and ``k`` the call is the reference's ``fftconv_bwd(y_grad, x_f, k_f,
    k_dtype)``."""
    if x.is_complex() or k.is_complex():
        return _fftconv_bwd_spectral(y_grad, x, k, k_dtype)
    dev = _require_cuda(y_grad, x, k)
    B, D, L = x.shape
    if y_grad.shape != x.shape or y_grad.dtype != x.dtype:
        raise RuntimeError("fftconv_bwd: y_grad must match x in shape and dtype")
    if x.dtype == torch.float64:
        dx, dk = _fftconv_f64_bwd(y_grad, x, k)
        return dx, dk.to(k_dtype)
    if L > fftconv_max_length():
        dx, dk = _fftconv_long_bwd(y_grad, x, k)
        return dx, dk.to(k_dtype)
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


# The reference's operator signatures (megalodon/csrc/ops/fftconv.cc:10-19,
# called from fused_ops/fftconv.py:79-106): the kernel arrives as the spectrum
# k_f = rfft(k, n=2M) (D, M+1), M = L rounded up to a power of two, unnormalised,
# and the forward hands back x_f = rfft(x, n=2M) (B, D, M+1) complex64 for the
# backward to keep.  The convolution kernels here work from the time-domain rows,
# so a spectrum is taken back to its row once on entry (exact up to float32
# rounding: the row was zero padded to 2M before it was transformed, so its first
# L samples are the row) and x_f is produced for the caller as the reference does.
def _spectrum_to_row(s: torch.Tensor, L: int, what: str) -> torch.Tensor:
    M = 1 << max(0, (L - 1).bit_length())
    if not s.is_complex() or s.shape[-1] != M + 1:
        raise RuntimeError(f"fftconv: {what} must be the complex spectrum of {M + 1} bins of rows of length {L}, "
                           f"got {tuple(s.shape)} {s.dtype}")
    wide = s.dtype == torch.complex128   # the double-precision flavour keeps its spectra in complex128
    return torch.fft.irfft(s if wide else s.to(torch.complex64), n=2 * M)[..., :L].contiguous()


def _fftconv_fwd_spectral(x: torch.Tensor, k_f: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    _require_cuda(x, k_f)
    L = x.shape[-1]
    M = 1 << max(0, (L - 1).bit_length())
    y = fftconv_fwd(x, _spectrum_to_row(k_f, L, "k_f"))
    if x.dtype == torch.float64:
        return y, torch.fft.rfft(x, n=2 * M)
    x_f = rfft(x, False) if 32 <= M <= 16384 else torch.fft.rfft(x.float(), n=2 * M)
    return y, x_f


def _fftconv_bwd_spectral(y_grad: torch.Tensor, x_f: torch.Tensor, k_f: torch.Tensor,
                          k_dtype: torch.dtype) -> Tuple[torch.Tensor, torch.Tensor]:
    _require_cuda(y_grad, x_f, k_f)
    L = y_grad.shape[-1]
    x = _spectrum_to_row(x_f, L, "x_f").to(y_grad.dtype)
    return fftconv_bwd(y_grad, x, _spectrum_to_row(k_f, L, "k_f"), k_dtype)


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
    if x.dtype == torch.float64:
        return _fftconv_f64_fwd(x, k) + x * omega.reshape(-1, 1).double()
    if L > fftconv_max_length():  # blocks, then the skip term in float32
        y = _fftconv_long_fwd(x, k).float() + x.float() * omega.reshape(-1, 1).float()
        return y.to(x.dtype)
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
    if x.dtype == torch.float64:
        dx, dk = _fftconv_f64_bwd(y_grad, x, k)
        return dx + y_grad * omega.reshape(-1, 1).double(), dk, dk[:, 0].clone()
    if L > fftconv_max_length():
        dx, dk = _fftconv_long_bwd(y_grad, x, k)
        dx = (dx.float() + y_grad.float() * omega.reshape(-1, 1).float()).to(x.dtype)
        return dx, dk, (y_grad.float() * x.float()).sum(dim=(0, 2))
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


def fftconv_prepare(L: int, device=None, stream=None) -> None:
    """Make the float32 convolution engine's tables and a scratch block for rows of
    L samples ahead of time, for `stream` (a torch.cuda.Stream; default: the current
    stream).  It allocates and synchronises once; later convolution calls on that
    stream only enqueue -- which is what a graph capture on that stream needs:
        fftconv_prepare(L, stream=s);  with torch.cuda.graph(g, stream=s): ..."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    if stream is not None:
        dev = stream.device
    with torch.cuda.device(dev):
        ptr = _lib.stream_ptr(dev) if stream is None else _lib.ctypes.c_void_p(stream.cuda_stream)
        _lib.call("mega_fftconv_prepare", _lib.i64(min(int(L), fftconv_max_length())), ptr)


def fftconv_scratch_blocks(L: int, device=None) -> int:
    """Scratch blocks the float32 convolution engine holds on `device` for the
    transform size of rows of L samples (at most four plus those owned by graphs)."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    with torch.cuda.device(dev):
        fn = _lib.load().mega_fftconv_scratch_blocks
        fn.restype = _lib.ctypes.c_int
        return int(fn(_lib.i64(int(L))))


def fftconv_spectrum_bytes(dtype: torch.dtype, B: int, D: int, L: int) -> int:
    """Bytes of one saved-spectrum buffer for this shape, 0 when the shape does
    not take the saved-spectrum path."""
    if dtype not in (torch.bfloat16, torch.float16):
        return 0
    fn = _lib.load().mega_fftconv_spectrum_bytes
    fn.restype = _lib.ctypes.c_int64
    return int(fn(_lib.i32(_lib.dtype_code(dtype)), _lib.i64(B), _lib.i64(D), _lib.i64(L)))


def fftconv_residual_fwd_saving(x: torch.Tensor, k: torch.Tensor, omega: torch.Tensor):
    """(y, spec_x, spec_k): ``fftconv_residual_fwd`` that also keeps the spectra
    of x and k for ``fftconv_residual_bwd_saved`` (the reference keeps x_f and
    k_f the same way, fused_ops/fftconv.py:21-28).  Only for shapes with
    ``fftconv_spectrum_bytes(...) > 0``."""
    dev = _require_cuda(x, k, omega)
    B, D, L = x.shape
    nbytes = fftconv_spectrum_bytes(x.dtype, B, D, L)
    if nbytes == 0:
        raise RuntimeError("fftconv: this shape / dtype has no saved-spectrum path")
    xc = x.contiguous()
    kc = k.contiguous().float()
    wc = omega.reshape(-1).contiguous().float()
    y = torch.empty_like(xc)
    spec_x = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    # the spectrum of k is kept once per channel, whatever the batch size
    spec_k = torch.empty(fftconv_spectrum_bytes(x.dtype, 1, D, L), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_fftconv_residual_fwd_saving", _lib.ptr(xc), _lib.i32(_lib.dtype_code(x.dtype)),
                  _lib.ptr(kc), _lib.ptr(wc), _lib.i64(B), _lib.i64(D), _lib.i64(L), _lib.ptr(y),
                  _lib.ptr(spec_x), _lib.ptr(spec_k), _lib.stream_ptr(dev))
    return y, spec_x, spec_k


def fftconv_residual_bwd_saved(y_grad: torch.Tensor, spec_x: torch.Tensor, spec_k: torch.Tensor,
                               omega: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dx, dk, domega) from y_grad (B, D, L) and the two saved spectra."""
    dev = _require_cuda(y_grad, spec_x, spec_k, omega)
    B, D, L = y_grad.shape
    if (spec_x.numel() != fftconv_spectrum_bytes(y_grad.dtype, B, D, L)
            or spec_k.numel() != fftconv_spectrum_bytes(y_grad.dtype, 1, D, L)):
        raise RuntimeError("fftconv_bwd: the saved spectra do not belong to this shape")
    dy = y_grad.contiguous()
    if dy.data_ptr() % 16 != 0:
        # a contiguous view at an odd storage offset: the kernel's 16-byte loads need an aligned row
        dy = dy.clone(memory_format=torch.contiguous_format)
    wc = omega.reshape(-1).contiguous().float()
    dx = torch.empty_like(dy)
    dk = torch.empty((D, L), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_fftconv_residual_bwd_saved", _lib.ptr(dy), _lib.i32(_lib.dtype_code(dy.dtype)),
                  _lib.ptr(spec_x), _lib.ptr(spec_k), _lib.ptr(wc), _lib.i64(B), _lib.i64(D), _lib.i64(L),
                  _lib.ptr(dx), _lib.ptr(dk), _lib.stream_ptr(dev))
    return dx, dk, dk[:, 0].clone()


# --------------------------------------------------------------------------
# The CEMA layer as a chunked recurrence (csrc/cema_scan.hip)
# --------------------------------------------------------------------------
def cema_scan_supported(x: torch.Tensor, ndim: int) -> bool:
    """Whether `cema_scan_fwd` takes this input: bfloat16 / float16 / float32 rows
    on the GPU, at most 32 modes (16 per launch), a length that is a multiple of 8."""
    if not x.is_cuda or x.dim() != 3 or x.dtype not in (torch.bfloat16, torch.float16, torch.float32) or ndim > 32:
        return False
    fn = _lib.load().mega_cema_scan_supported
    return bool(fn(_lib.i32(_lib.dtype_code(x.dtype)), _lib.i64(min(ndim, 16)), _lib.i64(x.shape[-1])))


def cema_scan_fwd(x: torch.Tensor, p: torch.Tensor, log_q: torch.Tensor, gamma: torch.Tensor,
                  omega: Optional[torch.Tensor], h0: Optional[torch.Tensor] = None,
                  compute_last_state: bool = False) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """(out, h_last): ``fftconv(x, k) + x * omega + b`` and, on request, the state
    after the last step, for k, b = ema_parameters(p, q, gamma, h0, L) -- without
    forming k (complex_exponential_moving_average.py:127-147).  x (B, D, L)
    bfloat16 / float16 / float32 (float32 rows enter the products with their 16
    leading bits, the precision the parameter matrices carry too: 1e-5 of the
    output's scale); p (D, N[, 1]) float32; log_q, gamma (D, N[, 1]) complex64."""
    dev = _require_cuda(x, p, log_q, gamma, omega, h0)
    B, D, L = x.shape
    N = p.shape[1]
    xc = x.contiguous()
    if xc.data_ptr() % 16 != 0:
        xc = xc.clone(memory_format=torch.contiguous_format)
    pc = p.reshape(D, N).contiguous().float()
    lq, gm = _as_c64(log_q, "log_q").reshape(D, N), _as_c64(gamma, "gamma").reshape(D, N)
    wc = None if omega is None else omega.reshape(-1).contiguous().float()
    hc = None if h0 is None else _as_c64(h0, "h0").reshape(B, D, N).contiguous()
    if N > 16:
        # mode groups of at most 16: the outputs add up (float32 sum, one rounding), the states are per mode
        ys, hs = None, []
        for i, (lo, hi) in enumerate(_mode_groups(N)):
            yi, hi_ = cema_scan_fwd(xc, pc[:, lo:hi], lq[:, lo:hi], gm[:, lo:hi], wc if i == 0 else None,
                                    None if hc is None else hc[:, :, lo:hi], compute_last_state)
            ys = yi.float() if ys is None else ys.add_(yi.float())
            hs.append(hi_)
        return ys.to(x.dtype), (torch.cat(hs, dim=2) if compute_last_state else None)
    y = torch.empty_like(xc)
    h_last = torch.empty((B, D, N), dtype=torch.complex64, device=dev) if compute_last_state else None
    with torch.cuda.device(dev):
        _lib.call("mega_cema_scan_fwd", _lib.ptr(xc), _lib.i32(_lib.dtype_code(x.dtype)), _lib.ptr(pc),
                  _lib.ptr(lq), _lib.ptr(gm), _lib.ptr(wc), _lib.ptr(hc), _lib.i64(B), _lib.i64(D), _lib.i64(N),
                  _lib.i64(L), _lib.ptr(y), _lib.ptr(h_last), _lib.stream_ptr(dev))
    return y, h_last


def cema_scan_bwd_supported(x: torch.Tensor, ndim: int) -> bool:
    """Whether the layer should train through `cema_scan_bwd` for this input: bfloat16
    rows (one launch), float16 and float32 rows (three launches on their two bfloat16
    pieces: 16 significant bits, what the forward takes of float32 rows as well);
    otherwise as the forward."""
    if not x.is_cuda or x.dim() != 3 or x.dtype not in (torch.bfloat16, torch.float16, torch.float32) or ndim > 32:
        return False
    fn = _lib.load().mega_cema_scan_bwd_supported
    return bool(fn(_lib.i32(_lib.dtype_code(torch.bfloat16)), _lib.i64(min(ndim, 16)), _lib.i64(x.shape[-1])))


def split_bf16(t: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """A float32 / float16 tensor as the sum of two bfloat16 tensors, hi = bf16(t) and
    lo = bf16(t - hi): 16 significant bits of a float32 value (what the recurrence's forward
    takes of float32 rows), every bit of a float16 one; one streaming kernel."""
    dev = _require_cuda(t)
    tc = t.contiguous()
    if tc.numel() % 8 != 0 or tc.data_ptr() % 16 != 0 or tc.dtype not in (torch.float32, torch.float16):
        hi = tc.to(torch.bfloat16)
        return hi, (tc.float() - hi.float()).to(torch.bfloat16)
    hi = torch.empty(tc.shape, dtype=torch.bfloat16, device=dev)
    lo = torch.empty_like(hi)
    with torch.cuda.device(dev):
        _lib.call("mega_split_bf16", _lib.ptr(tc), _lib.i32(_lib.dtype_code(tc.dtype)), _lib.i64(tc.numel()),
                  _lib.ptr(hi), _lib.ptr(lo), _lib.stream_ptr(dev))
    return hi, lo


def _cema_scan_bwd_wide(dy, x, pc, lq, gm, wc, hc, dx: Optional[torch.Tensor], accumulate: bool):
    """One launch of the backward kernel on bfloat16 pieces: float32 dx written, added to, or
    (None) left out; per-row parameter gradients summed over the batch; dh0 (or none)."""
    dev = x.device
    B, D, L = x.shape
    N = pc.shape[1]
    dp = torch.empty((B, D, N), dtype=torch.float32, device=dev)
    dq = torch.empty((B, D, N), dtype=torch.complex64, device=dev)
    dg = torch.empty((B, D, N), dtype=torch.complex64, device=dev)
    dw = torch.empty((B, D), dtype=torch.float32, device=dev)
    dh = None if hc is None else torch.empty((B, D, N), dtype=torch.complex64, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_cema_scan_bwd_wide", _lib.ptr(dy), _lib.ptr(x), _lib.ptr(pc), _lib.ptr(lq), _lib.ptr(gm),
                  _lib.ptr(wc), _lib.ptr(hc), _lib.i64(B), _lib.i64(D), _lib.i64(N), _lib.i64(L), _lib.ptr(dx),
                  _lib.i32(1 if accumulate else 0), _lib.ptr(dp), _lib.ptr(dq), _lib.ptr(dg), _lib.ptr(dw),
                  _lib.ptr(dh), _lib.stream_ptr(dev))
    return [dp.sum(0), dq.sum(0), dg.sum(0), dw.sum(0)], dh


def _mode_groups(N: int):
    """The kernels hold 16 modes; the modes of a channel are independent and their outputs add up,
    so more (the reference allows N <= 32, ema_parameters_kernel.cu:1026) run as several launches."""
    return [(lo, min(lo + 16, N)) for lo in range(0, N, 16)]


def cema_scan_bwd(y_grad: torch.Tensor, x: torch.Tensor, p: torch.Tensor, log_q: torch.Tensor,
                  gamma: torch.Tensor, omega: Optional[torch.Tensor], h0: Optional[torch.Tensor] = None):
    """(dx, dp, dq, dgamma, domega[, dh0]) of ``cema_scan_fwd(x, p, log_q, gamma, omega, h0)[0]``:
    dp (D, N) float32, dq and dgamma (D, N) complex64 in the convention of
    ``ema_parameters_bwd`` (gradient w.r.t. q, conjugated), domega (D,) float32 and,
    when a carried state h0 (B, D, N) is given, its gradient dh0 (B, D, N) complex64
    (ema_parameters.cc:158-188)."""
    dev = _require_cuda(y_grad, x, p, log_q, gamma, omega, h0)
    B, D, L = x.shape
    N = p.shape[1]
    if y_grad.shape != x.shape or y_grad.dtype != x.dtype:
        raise RuntimeError("cema_scan_bwd: y_grad must match x in shape and dtype")
    pc = p.reshape(D, N).contiguous().float()
    lq, gm = _as_c64(log_q, "log_q").reshape(D, N), _as_c64(gamma, "gamma").reshape(D, N)
    wc = None if omega is None else omega.reshape(-1).contiguous().float()
    hc = None if h0 is None else _as_c64(h0, "h0").reshape(B, D, N).contiguous()
    if N > 16:
        # mode groups of at most 16: dx and domega add up (the skip term rides on the first group),
        # the other gradients are per mode
        parts = []
        for i, (lo, hi) in enumerate(_mode_groups(N)):
            parts.append(cema_scan_bwd(y_grad, x, pc[:, lo:hi], lq[:, lo:hi], gm[:, lo:hi], wc if i == 0 else None,
                                       None if hc is None else hc[:, :, lo:hi]))
        dx = parts[0][0].float()
        for q_ in parts[1:]:
            dx += q_[0].float()
        out = [dx.to(x.dtype)] + [torch.cat([q_[j] for q_ in parts], dim=1) for j in (1, 2, 3)] + [parts[0][4]]
        if hc is not None:
            out.append(torch.cat([q_[5] for q_ in parts], dim=2))
        return tuple(out)
    if x.dtype != torch.bfloat16:
        # The backward is linear in y_grad and, for the parameter gradients, in x as well: the
        # bfloat16 kernel runs on the pairs of pieces (dy_hi, x_hi), (dy_lo, x_hi), (dy_hi, x_lo)
        # -- what is left out is 2^-16 of the result.  dx is linear in dy alone: the first two
        # launches write and add to it in float32, one rounding at the end; so the terms of a
        # carried state, which do not depend on x either.
        (g_hi, g_lo), (x_hi, x_lo) = split_bf16(y_grad), split_bf16(x)
        dx32 = torch.empty((B, D, L), dtype=torch.float32, device=dev)
        grads, dh = _cema_scan_bwd_wide(g_hi, x_hi, pc, lq, gm, wc, hc, dx32, False)
        g2, dh2 = _cema_scan_bwd_wide(g_lo, x_hi, pc, lq, gm, wc, hc, dx32, True)
        g3, _ = _cema_scan_bwd_wide(g_hi, x_lo, pc, lq, gm, wc, None, None, False)
        grads = [a_ + b_ + c_ for a_, b_, c_ in zip(grads, g2, g3)]
        out = (dx32 if x.dtype == torch.float32 else dx32.to(x.dtype), *grads)
        return out if hc is None else out + (dh + dh2,)

    def aligned(t):
        t = t.contiguous()
        return t if t.data_ptr() % 16 == 0 else t.clone(memory_format=torch.contiguous_format)

    dy, xc = aligned(y_grad), aligned(x)
    dx = torch.empty_like(xc)
    dp = torch.empty((B, D, N), dtype=torch.float32, device=dev)
    dq = torch.empty((B, D, N), dtype=torch.complex64, device=dev)
    dg = torch.empty((B, D, N), dtype=torch.complex64, device=dev)
    dw = torch.empty((B, D), dtype=torch.float32, device=dev)
    dh = None if hc is None else torch.empty((B, D, N), dtype=torch.complex64, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_cema_scan_bwd_state", _lib.ptr(dy), _lib.ptr(xc), _lib.i32(_lib.dtype_code(x.dtype)),
                  _lib.ptr(pc), _lib.ptr(lq), _lib.ptr(gm), _lib.ptr(wc), _lib.ptr(hc), _lib.i64(B), _lib.i64(D),
                  _lib.i64(N), _lib.i64(L), _lib.ptr(dx), _lib.ptr(dp), _lib.ptr(dq), _lib.ptr(dg), _lib.ptr(dw),
                  _lib.ptr(dh), _lib.stream_ptr(dev))
    out = (dx, dp[0], dq[0], dg[0], dw[0]) if B == 1 else (dx, dp.sum(0), dq.sum(0), dg.sum(0), dw.sum(0))
    return out if hc is None else out + (dh,)


# --------------------------------------------------------------------------
# group_timestep_norm (reference: csrc/ops/timestep_norm.cc:621-705)
# --------------------------------------------------------------------------
# One workspace per (device, stream, direction), grown on demand and kept: no
# allocation sits in the operator after its first call, and launches on
# different streams never share one (each call clears what it uses itself).
_tsn_ws_cache = {}


def _tsn_workspace(B, L, D, G, backward, dev):
    fn = _lib.load().mega_group_timestep_norm_workspace_bytes
    fn.restype = _lib.ctypes.c_int64
    nbytes = int(fn(_lib.i64(B), _lib.i64(L), _lib.i64(D), _lib.i64(G), _lib.i32(1 if backward else 0)))
    key = (dev.index if dev.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(dev).cuda_stream, bool(backward))
    ws = _tsn_ws_cache.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        _tsn_ws_cache[key] = ws
    return ws


def timestep_norm_status(device=None) -> None:
    """Waits for the current stream of `device` and raises RuntimeError if a tile
    of the last group_timestep_norm_fwd / _bwd launched on it gave up waiting for
    an earlier tile's statistics (its outputs are NaN then).  The kernels bound
    that wait themselves, so a launch always finishes; this call says whether
    one of them ran into the bound."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    idx = dev.index if dev.index is not None else torch.cuda.current_device()
    stream = torch.cuda.current_stream(dev).cuda_stream
    with torch.cuda.device(dev):
        for backward in (False, True):
            ws = _tsn_ws_cache.get((idx, stream, backward))
            if ws is not None:
                _lib.call("mega_group_timestep_norm_status", _lib.ptr(ws), _lib.stream_ptr(dev))


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
    stats_time_last: bool = False,
):
    """(y, count, mean, var, cummean, cumrstd); tensors other than count /
    mask / the statistics must share x's dtype, as in the reference
    (timestep_norm_kernel.cu:1270-1273); cummean and cumrstd are float32, float64
    for float64 x (the accumulate type, :1553-1565).

    `stats_time_last`: cummean and cumrstd come back as (B, G, L) instead of the
    reference's (B, L, G) -- for a caller that hands them to
    group_timestep_norm_bwd (with the same flag) and nowhere else, as the autograd
    node of the module does: a wavefront owns 64 steps of one group, so in that
    layout it writes and reads the statistics as whole lines (not available for
    float64 x)."""
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
    stat_dtype = torch.float64 if x.dtype == torch.float64 else torch.float32
    if stats_time_last and x.dtype == torch.float64:
        raise RuntimeError("stats_time_last is not available for float64 x")
    stat_shape = (B, G, L) if stats_time_last else (B, L, G)
    cummean = torch.empty(stat_shape, dtype=stat_dtype, device=dev)
    cumrstd = torch.empty(stat_shape, dtype=stat_dtype, device=dev)
    mask = _mask_bytes(padding_mask)
    if x.dtype == torch.float64:
        # the double-precision flavour: one wavefront per (batch, group) chain, no workspace
        if D % G != 0:
            raise RuntimeError("feature count must be a multiple of num_groups")
        with torch.cuda.device(dev):
            _lib.call("mega_group_timestep_norm_fwd_f64", _lib.ptr(xc), _lib.ptr(prev_count.contiguous()),
                      _lib.ptr(prev_mean.contiguous()), _lib.ptr(prev_var.contiguous()), _lib.ptr(gamma.contiguous()),
                      _lib.ptr(beta.contiguous()), _lib.ptr(mask), _lib.i64(B), _lib.i64(L), _lib.i64(D), _lib.i64(G),
                      _lib.f64(eps), _lib.ptr(y), _lib.ptr(count), _lib.ptr(mean), _lib.ptr(var), _lib.ptr(cummean),
                      _lib.ptr(cumrstd), _lib.stream_ptr(dev))
        return y, count, mean, var, cummean, cumrstd
    ws = _tsn_workspace(B, L, D, G, False, dev)
    with torch.cuda.device(dev):
        _lib.call("mega_group_timestep_norm_fwd_tl" if stats_time_last else "mega_group_timestep_norm_fwd",
                  _lib.ptr(xc), _lib.i32(_lib.dtype_code(x.dtype)),
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
    stats_time_last: bool = False,
):
    """(dx, dprev_mean, dprev_var, dgamma, dbeta).  `stats_time_last`: cummean and
    cumrstd are (B, G, L), as group_timestep_norm_fwd returns them under the same flag."""
    dev = _require_cuda(y_grad, mean_grad, var_grad, x, prev_mean, count, cummean, cumrstd, gamma, padding_mask)
    B, L, D = x.shape
    G = int(num_groups)
    want = (B, G, L) if stats_time_last else (B, L, G)
    if tuple(cummean.shape) != want or tuple(cumrstd.shape) != want:
        raise RuntimeError(f"cummean / cumrstd must be {want} (got {tuple(cummean.shape)}, {tuple(cumrstd.shape)})")
    if stats_time_last and x.dtype == torch.float64:
        raise RuntimeError("stats_time_last is not available for float64 x")
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
    if x.dtype == torch.float64:
        if cummean.dtype != torch.float64 or cumrstd.dtype != torch.float64:
            raise RuntimeError("cummean / cumrstd of float64 x must be float64")
        ws = torch.empty((2, B, D), dtype=torch.float64, device=dev)
        with torch.cuda.device(dev):
            _lib.call("mega_group_timestep_norm_bwd_f64", _lib.ptr(dy), _lib.ptr(mean_grad.contiguous()),
                      _lib.ptr(var_grad.contiguous()), _lib.ptr(xc), _lib.ptr(prev_mean.contiguous()),
                      _lib.ptr(count.contiguous()), _lib.ptr(cummean.contiguous()), _lib.ptr(cumrstd.contiguous()),
                      _lib.ptr(gamma.contiguous()), _lib.ptr(mask), _lib.i64(B), _lib.i64(L), _lib.i64(D), _lib.i64(G),
                      _lib.ptr(dx), _lib.ptr(dpm), _lib.ptr(dpv), _lib.ptr(dg), _lib.ptr(db), _lib.ptr(ws),
                      _lib.stream_ptr(dev))
        return dx, dpm, dpv, dg, db
    ws = _tsn_workspace(B, L, D, G, True, dev)
    with torch.cuda.device(dev):
        _lib.call("mega_group_timestep_norm_bwd_tl" if stats_time_last else "mega_group_timestep_norm_bwd",
                  _lib.ptr(dy), _lib.ptr(mean_grad.contiguous()),
                  _lib.ptr(var_grad.contiguous()), _lib.ptr(xc), _lib.i32(_lib.dtype_code(x.dtype)),
                  _lib.ptr(prev_mean.contiguous()), _lib.ptr(count.contiguous()),
                  _lib.ptr(cummean.contiguous()), _lib.ptr(cumrstd.contiguous()), _lib.ptr(gamma.contiguous()),
                  _lib.ptr(mask), _lib.i64(B), _lib.i64(L), _lib.i64(D), _lib.i64(G), _lib.ptr(dx),
                  _lib.ptr(dpm), _lib.ptr(dpv), _lib.ptr(dg), _lib.ptr(db), _lib.ptr(ws),
                  _lib.stream_ptr(dev))
    return dx, dpm, dpv, dg, db


def stream_copy(a: torch.Tensor, b: Optional[torch.Tensor] = None, workgroups: int = 8192,
                nontemporal: bool = False) -> torch.Tensor:
    """out = a (or a XOR b, bytewise) through the library's streaming reference
    kernel: the rate a kernel reaches that only moves an operator's bytes."""
    dev = _require_cuda(a, b)
    ac = a.contiguous()
    out = torch.empty_like(ac)
    nbytes = ac.numel() * ac.element_size()
    if b is not None and (b.shape != a.shape or b.dtype != a.dtype):
        raise RuntimeError("stream_copy: b must match a")
    bc = None if b is None else b.contiguous()
    with torch.cuda.device(dev):
        _lib.call("mega_bench_stream_copy", _lib.ptr(ac), _lib.ptr(bc), _lib.ptr(out), _lib.i64(nbytes),
                  _lib.i32(int(workgroups)), _lib.i32(1 if nontemporal else 0), _lib.stream_ptr(dev))
    return out


# --------------------------------------------------------------------------
# attention (reference: csrc/ops/attention.cc:28-29, attention_kernel.cu:261-303)
# --------------------------------------------------------------------------
def _attn_workspace(B, L1, L2, NH, H1, H2, backward, dev, dtype=torch.bfloat16):
    # the size query describes the 16-bit layout: float32 / float64 tensors need 2 / 4 times the bytes
    fn = _lib.load().mega_attention_workspace_bytes
    fn.restype = _lib.ctypes.c_int64
    nbytes = int(fn(_lib.i64(B), _lib.i64(L1), _lib.i64(L2), _lib.i64(NH), _lib.i64(H1), _lib.i64(H2),
                    _lib.i32(1 if backward else 0)))
    return torch.empty(nbytes * max(1, dtype.itemsize // 2), dtype=torch.uint8, device=dev)


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


def dropkey_philox_state(dev: torch.device, columns: int) -> Tuple[int, int]:
    """(seed, offset) for one DropKey launch, taken from PyTorch's generator of
    the device the way the reference does (attention_kernel.cu:100-109:
    `philox_cuda_state(capacity)`): the offset is read and then advanced, so
    successive launches draw different masks and `torch.manual_seed` /
    `torch.cuda.set_rng_state` reproduce them."""
    index = dev.index if dev.index is not None else torch.cuda.current_device()
    gen = torch.cuda.default_generators[index]
    seed, offset = gen.initial_seed(), gen.get_offset()
    gen.set_offset(offset + 4 * max(1, (columns + 3) // 4))
    return seed & 0xFFFFFFFFFFFFFFFF, offset


def attention_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, dropout: float,
                  use_causal_mask: bool, lower_only: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """(y, w): y (B, L1, N, H2), w = softmax probabilities (B, N, L1, L2), every
    row written to its end (zeros behind the causal limit, as the reference's
    softmax writes them, softmax.cuh:99-105,127-129).
    `dropout` > 0 is DropKey (softmax.cuh:135-196): keys leave a row with that
    probability before the softmax, drawn from the device generator's
    (seed, offset).  `lower_only` (no counterpart in the reference) is for callers
    that hand w to `attention_bwd` and nowhere else: with a causal mask and 16-bit
    tensors the zeros to the right of the block that holds a row's diagonal are
    then not written (half of w at L1 = L2), and those entries are undefined."""
    dev = _require_cuda(q, k, v)
    if not 0.0 <= dropout <= 1.0:
        raise RuntimeError("attention_fwd: dropout must lie in [0, 1]")
    B, L1, L2, NH, H1, H2 = _attn_dims(q, k, v)
    causal = (2 if lower_only else 1) if use_causal_mask else 0
    if dropout > 0.0:
        qc, kc, vc = q.contiguous(), k.contiguous(), v.contiguous()
        y = torch.empty((B, L1, NH, H2), dtype=v.dtype, device=dev)
        w = torch.empty((B, NH, L1, L2), dtype=v.dtype, device=dev)
        ws = _attn_workspace(B, L1, L2, NH, H1, H2, False, dev, q.dtype)
        seed, offset = dropkey_philox_state(dev, L2)
        with torch.cuda.device(dev):
            _lib.call("mega_attention_dropkey_fwd", _lib.ptr(qc), _lib.ptr(kc), _lib.ptr(vc),
                      _lib.i32(_lib.dtype_code(q.dtype, True)), _lib.i64(B), _lib.i64(L1), _lib.i64(L2),
                      _lib.i64(NH), _lib.i64(H1), _lib.i64(H2), _lib.f64(scale),
                      _lib.i32(causal), _lib.f64(dropout), _lib.u64(seed),
                      _lib.u64(offset), _lib.ptr(y), _lib.ptr(w), _lib.ptr(ws), _lib.stream_ptr(dev))
        return y, w
    qc, kc, vc = q.contiguous(), k.contiguous(), v.contiguous()
    y = torch.empty((B, L1, NH, H2), dtype=v.dtype, device=dev)
    w = torch.empty((B, NH, L1, L2), dtype=v.dtype, device=dev)
    ws = _attn_workspace(B, L1, L2, NH, H1, H2, False, dev, q.dtype)
    with torch.cuda.device(dev):
        _lib.call("mega_attention_fwd", _lib.ptr(qc), _lib.ptr(kc), _lib.ptr(vc),
                  _lib.i32(_lib.dtype_code(q.dtype, True)), _lib.i64(B), _lib.i64(L1), _lib.i64(L2), _lib.i64(NH),
                  _lib.i64(H1), _lib.i64(H2), _lib.f64(scale), _lib.i32(causal),
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
    ws = _attn_workspace(B, L1, L2, NH, H1, H2, True, dev, q.dtype)
    with torch.cuda.device(dev):
        _lib.call("mega_attention_bwd", _lib.ptr(dy), _lib.ptr(qc), _lib.ptr(kc), _lib.ptr(vc), _lib.ptr(wc),
                  _lib.i32(_lib.dtype_code(q.dtype, True)), _lib.i64(B), _lib.i64(L1), _lib.i64(L2), _lib.i64(NH),
                  _lib.i64(H1), _lib.i64(H2), _lib.f64(scale), _lib.i32(1 if use_causal_mask else 0),
                  _lib.ptr(dq), _lib.ptr(dk), _lib.ptr(dv), _lib.ptr(ws), _lib.stream_ptr(dev))
    return dq, dk, dv


def linear_weight_grad(y_grad: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """dW (out, in) = y_grad^T x for y_grad (tokens, out), x (tokens, in), bfloat16 / float16:
    the weight gradient of a linear layer on the attention operator's product kernel."""
    dev = _require_cuda(y_grad, x)
    if y_grad.dim() != 2 or x.dim() != 2 or y_grad.shape[0] != x.shape[0] or y_grad.dtype != x.dtype:
        raise RuntimeError("linear_weight_grad: y_grad (tokens, out) and x (tokens, in) of one dtype")
    g, xc = y_grad.contiguous(), x.contiguous()
    dw = torch.empty((g.shape[1], xc.shape[1]), dtype=x.dtype, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_linear_weight_grad", _lib.ptr(g), _lib.ptr(xc), _lib.i32(_lib.dtype_code(x.dtype)),
                  _lib.i64(g.shape[0]), _lib.i64(g.shape[1]), _lib.i64(xc.shape[1]), _lib.ptr(dw), _lib.stream_ptr(dev))
    return dw


def _softmax_dims(x: torch.Tensor):
    if x.dim() < 2:
        raise RuntimeError("attention_softmax: x needs at least two dimensions")
    L1, L2 = x.shape[-2], x.shape[-1]
    Z = x.numel() // max(1, L1 * L2)
    return Z, L1, L2


def attention_softmax_fwd(x: torch.Tensor, dropout: float, use_causal_mask: bool) -> torch.Tensor:
    """y = softmax(x) over the last axis (float32 inside), rows masked causally
    (bottom-right aligned) when asked; x (..., L1, L2) bfloat16 / float16 / float32
    (attention_softmax_kernel.cu:96-108)."""
    dev = _require_cuda(x)
    if not 0.0 <= dropout <= 1.0:
        raise RuntimeError("attention_softmax_fwd: dropout must lie in [0, 1]")
    Z, L1, L2 = _softmax_dims(x)
    y = x.contiguous().clone()
    if dropout > 0.0:
        seed, offset = dropkey_philox_state(dev, L2)
        with torch.cuda.device(dev):
            _lib.call("mega_attention_softmax_dropkey_fwd", _lib.ptr(y), _lib.i32(_lib.dtype_code(x.dtype, True)),
                      _lib.i64(Z), _lib.i64(L1), _lib.i64(L2), _lib.i32(1 if use_causal_mask else 0),
                      _lib.f64(dropout), _lib.u64(seed), _lib.u64(offset), _lib.stream_ptr(dev))
        return y
    with torch.cuda.device(dev):
        _lib.call("mega_attention_softmax_fwd", _lib.ptr(y), _lib.i32(_lib.dtype_code(x.dtype, True)), _lib.i64(Z),
                  _lib.i64(L1), _lib.i64(L2), _lib.i32(1 if use_causal_mask else 0), _lib.stream_ptr(dev))
    return y


def attention_softmax_bwd(y_grad: torch.Tensor, y: torch.Tensor, use_causal_mask: bool) -> torch.Tensor:
    """x_grad = y o (y_grad - rowsum(y o y_grad)) (attention_softmax_kernel.cu:110-123)."""
    dev = _require_cuda(y_grad, y)
    if y_grad.shape != y.shape or y_grad.dtype != y.dtype:
        raise RuntimeError("attention_softmax_bwd: y_grad and y must have the same shape and dtype")
    Z, L1, L2 = _softmax_dims(y)
    yc = y.contiguous()
    dx = y_grad.contiguous().clone()
    with torch.cuda.device(dev):
        _lib.call("mega_attention_softmax_bwd", _lib.ptr(yc), _lib.ptr(dx), _lib.i32(_lib.dtype_code(y.dtype, True)),
                  _lib.i64(Z), _lib.i64(L1), _lib.i64(L2), _lib.i32(1 if use_causal_mask else 0),
                  _lib.stream_ptr(dev))
    return dx


def dropout(x: torch.Tensor, p: float, seed: int, offset: int) -> torch.Tensor:
    """x / (1 - p) where element e is kept, 0 elsewhere; the mask is a pure
    function of (seed, offset, e), so the same call on a gradient is the
    backward (replaces the generator replay of
    megalodon/modules/fused_ops/memory_efficient_dropout.py:60-96)."""
    dev = _require_cuda(x)
    xc = x.contiguous()
    y = torch.empty_like(xc)
    with torch.cuda.device(dev):
        _lib.call("mega_dropout", _lib.ptr(xc), _lib.i32(_lib.dtype_code(x.dtype)), _lib.i64(xc.numel()),
                  _lib.f64(p), _lib.u64(seed), _lib.u64(offset), _lib.ptr(y), _lib.stream_ptr(dev))
    return y


def transpose_last2(x: torch.Tensor) -> torch.Tensor:
    """(..., R, C) -> contiguous (..., C, R): what `x.transpose(-2, -1).contiguous()`
    returns, in one tiled pass (the BLD <-> BDL moves around the EMA convolution,
    megalodon/modules/moving_average_gated_attention.py:299-300,314)."""
    dev = _require_cuda(x)
    if x.dim() < 2:
        raise RuntimeError("transpose_last2: x needs at least two dimensions")
    xc = x.contiguous()
    R, C = xc.shape[-2], xc.shape[-1]
    out = torch.empty(xc.shape[:-2] + (C, R), dtype=x.dtype, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_transpose", _lib.ptr(xc), _lib.i32(_lib.dtype_code(x.dtype)),
                  _lib.i64(xc.numel() // max(1, R * C)), _lib.i64(R), _lib.i64(C), _lib.ptr(out),
                  _lib.stream_ptr(dev))
    return out


def silu_mul_fwd(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """silu(a) * b (normalized_feedforward_network.py:82,
    moving_average_gated_attention.py:333-336), float32 inside."""
    dev = _require_cuda(a, b)
    if a.shape != b.shape or a.dtype != b.dtype:
        raise RuntimeError("silu_mul: a and b must have the same shape and dtype")
    ac, bc = a.contiguous(), b.contiguous()
    out = torch.empty_like(ac)
    with torch.cuda.device(dev):
        _lib.call("mega_silu_mul_fwd", _lib.ptr(ac), _lib.ptr(bc), _lib.i32(_lib.dtype_code(a.dtype)),
                  _lib.i64(ac.numel()), _lib.ptr(out), _lib.stream_ptr(dev))
    return out


def silu_mul_bwd(out_grad: torch.Tensor, a: torch.Tensor, b: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """(a_grad, b_grad) of silu(a) * b."""
    dev = _require_cuda(out_grad, a, b)
    if not (out_grad.shape == a.shape == b.shape) or not (out_grad.dtype == a.dtype == b.dtype):
        raise RuntimeError("silu_mul_bwd: out_grad, a and b must have the same shape and dtype")
    gc, ac, bc = out_grad.contiguous(), a.contiguous(), b.contiguous()
    da, db = torch.empty_like(ac), torch.empty_like(bc)
    with torch.cuda.device(dev):
        _lib.call("mega_silu_mul_bwd", _lib.ptr(gc), _lib.ptr(ac), _lib.ptr(bc), _lib.i32(_lib.dtype_code(a.dtype)),
                  _lib.i64(ac.numel()), _lib.ptr(da), _lib.ptr(db), _lib.stream_ptr(dev))
    return da, db


def layer_norm_fwd(x: torch.Tensor, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor], eps: float,
                   rms: bool) -> Tuple[torch.Tensor, Optional[torch.Tensor], torch.Tensor]:
    """(y, mean, rstd) of LayerNorm / RMSNorm over the last axis with the stored
    weight = gamma - 1 (megalodon/modules/layer_norm.py:30-33,62-65)."""
    dev = _require_cuda(x)
    D = x.shape[-1]
    for t, name in ((weight, "weight"), (bias, "bias")):
        if t is not None and (t.shape != (D,) or t.dtype != x.dtype or t.device != x.device):
            raise RuntimeError(f"layer_norm: {name} must be ({D},) of x's dtype on x's device")
    xc = x.contiguous()
    rows = xc.numel() // D
    y = torch.empty_like(xc)
    mean = None if rms else torch.empty(rows, dtype=torch.float32, device=dev)
    rstd = torch.empty(rows, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_layer_norm_fwd", _lib.ptr(xc), _lib.ptr(None if weight is None else weight.contiguous()),
                  _lib.ptr(None if bias is None or rms else bias.contiguous()), _lib.i32(_lib.dtype_code(x.dtype)),
                  _lib.i64(rows), _lib.i64(D), _lib.f64(eps), _lib.i32(1 if rms else 0), _lib.ptr(y),
                  _lib.ptr(mean), _lib.ptr(rstd), _lib.stream_ptr(dev))
    return y, mean, rstd


def layer_norm_bwd(y_grad: torch.Tensor, x: torch.Tensor, weight: Optional[torch.Tensor],
                   mean: Optional[torch.Tensor], rstd: torch.Tensor, rms: bool, has_bias: bool
                   ) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """(x_grad, weight_grad, bias_grad)."""
    dev = _require_cuda(y_grad, x)
    if y_grad.shape != x.shape or y_grad.dtype != x.dtype:
        raise RuntimeError("layer_norm_bwd: y_grad and x must have the same shape and dtype")
    D = x.shape[-1]
    xc, gc = x.contiguous(), y_grad.contiguous()
    rows = xc.numel() // D
    dx = torch.empty_like(xc)
    if rows == 0:
        return (dx, None if weight is None else torch.zeros_like(weight),
                torch.zeros(D, dtype=x.dtype, device=dev) if has_bias and not rms else None)
    dw = None if weight is None else torch.empty_like(weight)
    db = torch.empty(D, dtype=x.dtype, device=dev) if (has_bias and not rms and weight is not None) else None
    ws = None
    if dw is not None:
        fn = _lib.load().mega_layer_norm_workspace_bytes
        fn.restype = _lib.ctypes.c_int64
        ws = torch.empty(int(fn(_lib.i64(rows), _lib.i64(D))), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_layer_norm_bwd", _lib.ptr(gc), _lib.ptr(xc),
                  _lib.ptr(None if weight is None else weight.contiguous()), _lib.ptr(mean), _lib.ptr(rstd),
                  _lib.i32(_lib.dtype_code(x.dtype)), _lib.i64(rows), _lib.i64(D), _lib.i32(1 if rms else 0),
                  _lib.ptr(dx), _lib.ptr(dw), _lib.ptr(db), _lib.ptr(ws), _lib.stream_ptr(dev))
    return dx, dw, db


def qk_norm_rotary_supported(z: torch.Tensor, gamma: torch.Tensor, head_dim: int) -> bool:
    """Shapes the fused z -> (q, k) kernel takes (include/megalodon_hip.h)."""
    return (z.is_cuda and z.dtype in (torch.bfloat16, torch.float16) and gamma.dtype == z.dtype
            and head_dim in (64, 128, 256, 512) and z.shape[-1] in (512, 1024, 2048, 4096)
            and z.shape[-1] % head_dim == 0 and z.dim() == 3)


def _freqs_real(freqs_cis: Optional[torch.Tensor], head_dim: int, dev) -> Tuple[Optional[torch.Tensor], int]:
    if freqs_cis is None:
        return None, 1
    if freqs_cis.dim() != 2 or freqs_cis.shape[1] != head_dim // 2 or not freqs_cis.is_complex():
        raise RuntimeError("qk_norm_rotary: freqs_cis must be complex (positions, head_dim / 2)")
    fr = torch.view_as_real(freqs_cis.to(device=dev, dtype=torch.complex64)).contiguous()
    return fr, freqs_cis.shape[0]


def qk_norm_rotary_fwd(z: torch.Tensor, gamma: torch.Tensor, beta: torch.Tensor,
                       freqs_cis: Optional[torch.Tensor], head_dim: int, eps: float
                       ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(q, k, rstd) from z (B, L, S): RMSNorm per head, `* (gamma + 1) / sqrt(head_dim) + beta`
    for q and for k, rotary by position inside the chunk
    (moving_average_gated_attention.py:319-330, rotary_positional_embedding.py:53-77)."""
    dev = _require_cuda(z, gamma, beta)
    if z.dim() != 3 or gamma.shape != (2, z.shape[-1]) or beta.shape != gamma.shape:
        raise RuntimeError("qk_norm_rotary: z must be (B, L, S), gamma and beta (2, S)")
    B, L, S = z.shape
    zc, gc, bc = z.contiguous(), gamma.contiguous(), beta.contiguous()
    fr, P = _freqs_real(freqs_cis, head_dim, dev)
    q, k = torch.empty_like(zc), torch.empty_like(zc)
    rstd = torch.empty(B * L, S // head_dim, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_qk_norm_rotary_fwd", _lib.ptr(zc), _lib.ptr(gc), _lib.ptr(bc), _lib.ptr(fr),
                  _lib.i32(_lib.dtype_code(z.dtype)), _lib.i64(B * L), _lib.i64(L), _lib.i64(P), _lib.i64(S),
                  _lib.i64(head_dim), _lib.f64(eps), _lib.ptr(q), _lib.ptr(k), _lib.ptr(rstd), _lib.stream_ptr(dev))
    return q, k, rstd


def qk_norm_rotary_bwd(q_grad: torch.Tensor, k_grad: torch.Tensor, z: torch.Tensor, gamma: torch.Tensor,
                       rstd: torch.Tensor, freqs_cis: Optional[torch.Tensor], head_dim: int
                       ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(z_grad, gamma_grad, beta_grad)."""
    dev = _require_cuda(q_grad, k_grad, z, gamma)
    B, L, S = z.shape
    zc, gc, dq, dk = z.contiguous(), gamma.contiguous(), q_grad.contiguous(), k_grad.contiguous()
    fr, P = _freqs_real(freqs_cis, head_dim, dev)
    dz, dgamma, dbeta = torch.empty_like(zc), torch.empty_like(gc), torch.empty_like(gc)
    fn = _lib.load().mega_qk_norm_rotary_workspace_bytes
    fn.restype = _lib.ctypes.c_int64
    ws = torch.empty(int(fn(_lib.i64(S))), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_qk_norm_rotary_bwd", _lib.ptr(dq), _lib.ptr(dk), _lib.ptr(zc), _lib.ptr(gc), _lib.ptr(rstd),
                  _lib.ptr(fr), _lib.i32(_lib.dtype_code(z.dtype)), _lib.i64(B * L), _lib.i64(L), _lib.i64(P),
                  _lib.i64(S), _lib.i64(head_dim), _lib.ptr(dz), _lib.ptr(dgamma), _lib.ptr(dbeta), _lib.ptr(ws),
                  _lib.stream_ptr(dev))
    return dz, dgamma, dbeta


def rfft(x: torch.Tensor, flip: bool = False) -> torch.Tensor:
    """`torch.fft.rfft(x, n=2 M)` over the last axis, M = max(2^ceil(log2 L), 32),
    on the (optionally time-reversed) rows; complex64 (..., M + 1)
    (megalodon/csrc/ops/fftconv.cc:6-8, fftconv_kernel.cu:170-215)."""
    dev = _require_cuda(x)
    L = x.shape[-1]
    xc = x.contiguous()
    rows = xc.numel() // max(1, L)
    fn = _lib.load().mega_rfft_bins
    fn.restype = _lib.ctypes.c_int64
    bins = int(fn(_lib.i64(L)))
    y = torch.empty(x.shape[:-1] + (bins,), dtype=torch.complex64, device=dev)
    with torch.cuda.device(dev):
        _lib.call("mega_rfft", _lib.ptr(xc), _lib.i32(_lib.dtype_code(x.dtype)), _lib.i64(rows), _lib.i64(L),
                  _lib.i32(1 if flip else 0), _lib.ptr(y), _lib.stream_ptr(dev))
    return y


def timestep_norm_fwd(x: torch.Tensor, prev_count: torch.Tensor, prev_mean: torch.Tensor, prev_var: torch.Tensor,
                      gamma: torch.Tensor, beta: torch.Tensor, padding_mask: Optional[torch.Tensor], eps: float):
    """The non-group operator (megalodon/csrc/ops/timestep_norm.cc:23-105,
    binding :700-701): every feature keeps its own running mean / variance,
    i.e. the group operator with one feature per group.  Returns (y, count,
    mean, var, cummean, cumrstd) with the saved statistics in x's dtype, as the
    reference does for this variant (:53-54).  The module path never calls it
    (modules/timestep_norm.py:123-125 always takes the group operator), so it
    runs on the general one-wave-per-chain kernel."""
    H = x.shape[-1]
    y, count, mean, var, cummean, cumrstd = group_timestep_norm_fwd(
        x, prev_count, prev_mean, prev_var, gamma, beta, padding_mask, H, eps)
    return y, count, mean, var, cummean.to(x.dtype), cumrstd.to(x.dtype)


def timestep_norm_bwd(y_grad: torch.Tensor, mean_grad: torch.Tensor, var_grad: torch.Tensor, x: torch.Tensor,
                      prev_mean: torch.Tensor, count: torch.Tensor, cummean: torch.Tensor, cumrstd: torch.Tensor,
                      gamma: torch.Tensor, padding_mask: Optional[torch.Tensor]):
    """(dx, dprev_mean, dprev_var, dgamma, dbeta) of the non-group operator
    (timestep_norm.cc:107-216, binding :702-703)."""
    H = x.shape[-1]
    return group_timestep_norm_bwd(y_grad, mean_grad, var_grad, x, prev_mean, count, cummean.float(),
                                   cumrstd.float(), gamma, padding_mask, H)


def _sequence_norm_geometry(x: torch.Tensor, gamma: torch.Tensor, padding_mask, num_groups: int, length_last: bool):
    if x.dim() != 3:
        raise RuntimeError("sequence_norm: x must be (B, L, H) or, with length_last, (B, H, L)")
    B = x.shape[0]
    L, H = (x.shape[2], x.shape[1]) if length_last else (x.shape[1], x.shape[2])
    if gamma.shape != (H,) or gamma.dtype != x.dtype:
        raise RuntimeError(f"sequence_norm: gamma and beta must be ({H},) of x's dtype")
    if num_groups < 1 or H % num_groups != 0:
        raise RuntimeError(f"sequence_norm: num_groups {num_groups} does not divide H={H}")
    if padding_mask is not None and padding_mask.shape != (B, L):
        raise RuntimeError(f"sequence_norm: padding_mask must be ({B}, {L})")
    return B, L, H


def _sequence_norm_workspace(dev, B, L, H, num_groups, length_last):
    fn = _lib.load().mega_group_sequence_norm_workspace_bytes
    fn.restype = _lib.ctypes.c_int64
    size = int(fn(_lib.i64(B), _lib.i64(L), _lib.i64(H), _lib.i64(num_groups), _lib.i32(1 if length_last else 0)))
    return torch.empty(max(size, 256), dtype=torch.uint8, device=dev)


def group_sequence_norm_fwd(x: torch.Tensor, gamma: torch.Tensor, beta: torch.Tensor,
                            padding_mask: Optional[torch.Tensor], num_groups: int, eps: float,
                            length_last: bool = False):
    """(y, count, mean, rstd): normalisation of every (sequence, feature group)
    over its unmasked steps and the group's features
    (megalodon/csrc/ops/sequence_norm.cc:953-1010, binding :1068-1069)."""
    dev = _require_cuda(x, gamma, beta, padding_mask)
    B, L, H = _sequence_norm_geometry(x, gamma, padding_mask, num_groups, length_last)
    if beta.shape != gamma.shape or beta.dtype != x.dtype:
        raise RuntimeError(f"sequence_norm: gamma and beta must be ({H},) of x's dtype")
    xc = x.contiguous()
    y = torch.empty_like(xc)
    count = torch.empty(B, dtype=torch.int64, device=dev)
    mean = torch.empty(B, num_groups, dtype=torch.float32, device=dev)
    rstd = torch.empty(B, num_groups, dtype=torch.float32, device=dev)
    mask = _mask_bytes(padding_mask)
    ws = _sequence_norm_workspace(dev, B, L, H, num_groups, length_last)
    with torch.cuda.device(dev):
        _lib.call("mega_group_sequence_norm_fwd", _lib.ptr(xc), _lib.ptr(gamma.contiguous()),
                  _lib.ptr(beta.contiguous()), _lib.ptr(mask), _lib.i32(_lib.dtype_code(x.dtype)), _lib.i64(B),
                  _lib.i64(L), _lib.i64(H), _lib.i64(num_groups), _lib.f64(eps), _lib.i32(1 if length_last else 0),
                  _lib.ptr(y), _lib.ptr(count), _lib.ptr(mean), _lib.ptr(rstd), _lib.ptr(ws), _lib.stream_ptr(dev))
    return y, count, mean, rstd


def group_sequence_norm_bwd(y_grad: torch.Tensor, x: torch.Tensor, count: torch.Tensor, mean: torch.Tensor,
                            rstd: torch.Tensor, gamma: torch.Tensor, padding_mask: Optional[torch.Tensor],
                            num_groups: int, length_last: bool = False):
    """(x_grad, gamma_grad, beta_grad)
    (megalodon/csrc/ops/sequence_norm.cc:1012-1063, binding :1070-1071)."""
    dev = _require_cuda(y_grad, x, count, mean, rstd, gamma, padding_mask)
    B, L, H = _sequence_norm_geometry(x, gamma, padding_mask, num_groups, length_last)
    if y_grad.shape != x.shape or y_grad.dtype != x.dtype:
        raise RuntimeError("sequence_norm_bwd: y_grad and x must have the same shape and dtype")
    if (count.shape != (B,) or count.dtype != torch.int64 or mean.shape != (B, num_groups)
            or rstd.shape != (B, num_groups) or mean.dtype != torch.float32 or rstd.dtype != torch.float32):
        raise RuntimeError("sequence_norm_bwd: count must be int64 (B,), mean and rstd float32 (B, num_groups)")
    xc, gc = x.contiguous(), y_grad.contiguous()
    dx = torch.empty_like(xc)
    dgamma = torch.empty_like(gamma, memory_format=torch.contiguous_format)
    dbeta = torch.empty_like(dgamma)
    mask = _mask_bytes(padding_mask)
    ws = _sequence_norm_workspace(dev, B, L, H, num_groups, length_last)
    with torch.cuda.device(dev):
        _lib.call("mega_group_sequence_norm_bwd", _lib.ptr(gc), _lib.ptr(xc), _lib.ptr(count.contiguous()),
                  _lib.ptr(mean.contiguous()), _lib.ptr(rstd.contiguous()), _lib.ptr(gamma.contiguous()),
                  _lib.ptr(mask), _lib.i32(_lib.dtype_code(x.dtype)), _lib.i64(B), _lib.i64(L), _lib.i64(H),
                  _lib.i64(num_groups), _lib.i32(1 if length_last else 0), _lib.ptr(dx), _lib.ptr(dgamma),
                  _lib.ptr(dbeta), _lib.ptr(ws), _lib.stream_ptr(dev))
    return dx, dgamma, dbeta


def sequence_norm_fwd(x: torch.Tensor, gamma: torch.Tensor, beta: torch.Tensor,
                      padding_mask: Optional[torch.Tensor], eps: float, length_last: bool = False):
    """The per-feature operator: one group per feature, statistics (B, H)
    (megalodon/csrc/ops/sequence_norm.cc:844-900, binding :1066)."""
    H = x.shape[1] if length_last else x.shape[-1]
    return group_sequence_norm_fwd(x, gamma, beta, padding_mask, H, eps, length_last)


def sequence_norm_bwd(y_grad: torch.Tensor, x: torch.Tensor, count: torch.Tensor, mean: torch.Tensor,
                      rstd: torch.Tensor, gamma: torch.Tensor, padding_mask: Optional[torch.Tensor],
                      length_last: bool = False):
    """(x_grad, gamma_grad, beta_grad) of the per-feature operator
    (megalodon/csrc/ops/sequence_norm.cc:902-951, binding :1067)."""
    H = x.shape[1] if length_last else x.shape[-1]
    return group_sequence_norm_bwd(y_grad, x, count, mean, rstd, gamma, padding_mask, H, length_last)
