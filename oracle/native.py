"""ctypes access to the compiled CPU checkers (TEST INFRASTRUCTURE ONLY).

``port()``  -> oracle/liboracle_cpu.so, the C/OpenMP restatement (oracle/cpu_ref.c)
``ref()``   -> oracle/_ref/libmegalodon_ref_cpu.so, the reference's own C++ CPU
               operators compiled from /root/reference (None when not built)
Both take and return float32 torch CPU tensors.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
PORT_PATH = os.path.join(HERE, "liboracle_cpu.so")
REF_PATH = os.path.join(HERE, "_ref", "libmegalodon_ref_cpu.so")

_port = None
_ref = None


def build(with_reference: bool = True) -> None:
    """Compile the checkers (make); the reference build is skipped when
    /root/reference is absent."""
    subprocess.run(["make", "-C", HERE, "liboracle_cpu.so"], check=True, capture_output=True)
    if with_reference:
        subprocess.run(["make", "-C", HERE, "ref"], check=True, capture_output=True)


def port() -> ctypes.CDLL:
    global _port
    if _port is None:
        if not os.path.exists(PORT_PATH):
            build(with_reference=False)
        _port = ctypes.CDLL(PORT_PATH)
    return _port


def ref() -> Optional[ctypes.CDLL]:
    global _ref
    if _ref is None and os.path.exists(REF_PATH):
        _ref = ctypes.CDLL(REF_PATH)
    return _ref


def _p(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _i(v):
    return ctypes.c_int64(int(v))


def _c64_as_f32(t):
    return torch.view_as_real(t.to(torch.complex64).contiguous().resolve_conj()).contiguous()


def ema_weight_fwd(lib, prefix, p, log_q, gamma, L):
    D = p.shape[0]
    pf = p.reshape(D, -1).float().contiguous()
    N = pf.shape[1]
    lq = _c64_as_f32(log_q.reshape(D, N))
    gm = _c64_as_f32(gamma.reshape(D, N))
    w = torch.empty(D, L, dtype=torch.float32)
    getattr(lib, prefix + "ema_weight_fwd")(_p(pf), _p(lq), _p(gm), _i(D), _i(N), _i(L), _p(w))
    return w


def ema_weight_bwd(lib, prefix, dw, p, log_q, gamma):
    D = p.shape[0]
    pf = p.reshape(D, -1).float().contiguous()
    N = pf.shape[1]
    L = dw.shape[-1]
    lq = _c64_as_f32(log_q.reshape(D, N))
    gm = _c64_as_f32(gamma.reshape(D, N))
    dwf = dw.float().contiguous()
    dp = torch.empty(D, N, dtype=torch.float32)
    dq = torch.empty(D, N, 2, dtype=torch.float32)
    dg = torch.empty(D, N, 2, dtype=torch.float32)
    getattr(lib, prefix + "ema_weight_bwd")(_p(dwf), _p(pf), _p(lq), _p(gm), _i(D), _i(N), _i(L),
                                            _p(dp), _p(dq), _p(dg))
    return dp, torch.view_as_complex(dq), torch.view_as_complex(dg)


def group_timestep_norm_fwd(lib, prefix, x, prev_count, prev_mean, prev_var, gamma, beta, mask, G, eps):
    B, L, H = x.shape
    xf = x.float().contiguous()
    pc = prev_count.to(torch.int64).contiguous()
    pm, pv = prev_mean.float().contiguous(), prev_var.float().contiguous()
    gm, bt = gamma.float().contiguous(), beta.float().contiguous()
    mk = None if mask is None else mask.to(torch.uint8).contiguous()
    y = torch.empty_like(xf)
    count = torch.empty(B, dtype=torch.int64)
    mean = torch.empty(B, G)
    var = torch.empty(B, G)
    cummean = torch.empty(B, L, G)
    cumrstd = torch.empty(B, L, G)
    getattr(lib, prefix + "group_timestep_norm_fwd")(
        _p(xf), _p(pc), _p(pm), _p(pv), _p(gm), _p(bt), _p(mk), _i(B), _i(L), _i(H), _i(G),
        ctypes.c_double(eps), _p(y), _p(count), _p(mean), _p(var), _p(cummean), _p(cumrstd))
    return y, count, mean, var, cummean, cumrstd


def group_timestep_norm_bwd(lib, prefix, dy, dmean, dvar, x, prev_mean, count, cummean, cumrstd, gamma, mask, G):
    B, L, H = x.shape
    dyf, xf = dy.float().contiguous(), x.float().contiguous()
    dm, dv = dmean.float().contiguous(), dvar.float().contiguous()
    pm = prev_mean.float().contiguous()
    cnt = count.to(torch.int64).contiguous()
    cm, cr = cummean.float().contiguous(), cumrstd.float().contiguous()
    gm = gamma.float().contiguous()
    mk = None if mask is None else mask.to(torch.uint8).contiguous()
    dx = torch.empty_like(xf)
    dpm = torch.empty(B, G)
    dpv = torch.empty(B, G)
    dg = torch.empty(H)
    db = torch.empty(H)
    getattr(lib, prefix + "group_timestep_norm_bwd")(
        _p(dyf), _p(dm), _p(dv), _p(xf), _p(pm), _p(cnt), _p(cm), _p(cr), _p(gm), _p(mk),
        _i(B), _i(L), _i(H), _i(G), _p(dx), _p(dpm), _p(dpv), _p(dg), _p(db))
    return dx, dpm, dpv, dg, db


# ---- carried state (reference build only) ---------------------------------------
def ema_bias_fwd(lib, p, log_q, gamma, h, L):
    B, D, N = h.shape
    pf = p.reshape(D, N).float().contiguous()
    b = torch.empty(B, D, L, dtype=torch.float32)
    lib.ref_ema_bias_fwd(_p(pf), _p(_c64_as_f32(log_q.reshape(D, N))), _p(_c64_as_f32(gamma.reshape(D, N))),
                         _p(_c64_as_f32(h)), _i(B), _i(D), _i(N), _i(L), _p(b))
    return b


def ema_bias_bwd(lib, db, p, log_q, gamma, h):
    B, D, N = h.shape
    L = db.shape[-1]
    pf = p.reshape(D, N).float().contiguous()
    dq = torch.empty(D, N, 2, dtype=torch.float32)
    dg = torch.empty(D, N, 2, dtype=torch.float32)
    dh = torch.empty(B, D, N, 2, dtype=torch.float32)
    lib.ref_ema_bias_bwd(_p(db.float().contiguous()), _p(pf), _p(_c64_as_f32(log_q.reshape(D, N))),
                         _p(_c64_as_f32(gamma.reshape(D, N))), _p(_c64_as_f32(h)), _i(B), _i(D), _i(N),
                         _i(L), _p(dq), _p(dg), _p(dh))
    return torch.view_as_complex(dq), torch.view_as_complex(dg), torch.view_as_complex(dh)


def ema_hidden_fwd(lib, x, p, log_q, h):
    B, D, L = x.shape
    pf = p.reshape(D, -1).float().contiguous()
    N = pf.shape[1]
    y = torch.empty(B, D, N, 2, dtype=torch.float32)
    lib.ref_ema_hidden_fwd(_p(x.float().contiguous()), _p(pf), _p(_c64_as_f32(log_q.reshape(D, N))),
                           _p(None if h is None else _c64_as_f32(h)), _i(B), _i(D), _i(N), _i(L), _p(y))
    return torch.view_as_complex(y)


def ema_hidden_bwd(lib, dy, x, p, log_q, h):
    B, D, L = x.shape
    pf = p.reshape(D, -1).float().contiguous()
    N = pf.shape[1]
    dx = torch.empty(B, D, L, dtype=torch.float32)
    dp = torch.empty(D, N, dtype=torch.float32)
    dq = torch.empty(D, N, 2, dtype=torch.float32)
    dh = torch.empty(B, D, N, 2, dtype=torch.float32)
    lib.ref_ema_hidden_bwd(_p(_c64_as_f32(dy)), _p(x.float().contiguous()), _p(pf),
                           _p(_c64_as_f32(log_q.reshape(D, N))), _p(None if h is None else _c64_as_f32(h)),
                           _i(B), _i(D), _i(N), _i(L), _p(dx), _p(dp), _p(dq), _p(dh))
    return dx, dp, torch.view_as_complex(dq), (None if h is None else torch.view_as_complex(dh))


# ---- whole-sequence group normalisation (reference build only) --------------------
def group_sequence_norm_fwd(lib, x, gamma, beta, mask, G, eps, length_last=False):
    B = x.shape[0]
    L, H = (x.shape[2], x.shape[1]) if length_last else (x.shape[1], x.shape[2])
    xf = x.float().contiguous()
    gm, bt = gamma.float().contiguous(), beta.float().contiguous()
    mk = None if mask is None else mask.to(torch.uint8).contiguous()
    y = torch.empty_like(xf)
    count = torch.empty(B, dtype=torch.int64)
    mean = torch.empty(B, G)
    rstd = torch.empty(B, G)
    lib.ref_group_sequence_norm_fwd(_p(xf), _p(gm), _p(bt), _p(mk), _i(B), _i(L), _i(H), _i(G), ctypes.c_double(eps),
                                    ctypes.c_int(1 if length_last else 0), _p(y), _p(count), _p(mean), _p(rstd))
    return y, count, mean, rstd


def group_sequence_norm_bwd(lib, dy, x, count, mean, rstd, gamma, mask, G, length_last=False):
    B = x.shape[0]
    L, H = (x.shape[2], x.shape[1]) if length_last else (x.shape[1], x.shape[2])
    dyf, xf = dy.float().contiguous(), x.float().contiguous()
    cnt = count.to(torch.int64).contiguous()
    mn, rs = mean.float().contiguous(), rstd.float().contiguous()
    gm = gamma.float().contiguous()
    mk = None if mask is None else mask.to(torch.uint8).contiguous()
    dx = torch.empty_like(xf)
    dg = torch.empty(H)
    db = torch.empty(H)
    lib.ref_group_sequence_norm_bwd(_p(dyf), _p(xf), _p(cnt), _p(mn), _p(rs), _p(gm), _p(mk), _i(B), _i(L), _i(H),
                                    _i(G), ctypes.c_int(1 if length_last else 0), _p(dx), _p(dg), _p(db))
    return dx, dg, db
