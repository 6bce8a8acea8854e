"""`ema_hidden(x, p, q, hx) -> h`: the EMA state after the last step of x (and
of a carried state `hx`), as the op of
megalodon/modules/fused_ops/ema_hidden.py:8-33."""
from .. import extension as ops
from ._autograd import fused_op


def _run(x, p, q, hx):
    log_q = q.log()
    h, vander = ops.ema_hidden_fwd(x, p, log_q, hx)
    return h, (x, p, log_q, hx, vander), None


def _grad(_, saved, h_grad):
    return ops.ema_hidden_bwd(h_grad, *saved)  # (dx, dp, dq, dhx)


EMAHiddenFunc = fused_op("EMAHiddenFunc", _run, _grad, doc=__doc__)
ema_hidden = EMAHiddenFunc.apply
