"""`ema_parameters(p, q, gamma, hx, length) -> (weight, bias)`: the CEMA
convolution kernel and, with a carried state `hx`, its bias rows, as the op of
megalodon/modules/fused_ops/ema_parameters.py:8-35.  The entry points work on
log q; the gradient comes back with respect to q itself."""
from .. import extension as ops
from ._autograd import fused_op


def _run(p, q, gamma, hx, length):
    log_q = q.log()
    weight, bias, vander = ops.ema_parameters_fwd(p, log_q, gamma, hx, length)
    return (weight, bias), (p, log_q, gamma, hx, vander), None


def _grad(_, saved, weight_grad, bias_grad):
    # (dp, dq, dgamma, dhx) + nothing for `length`
    return (*ops.ema_parameters_bwd(weight_grad, bias_grad, *saved), None)


EMAParametersFunc = fused_op("EMAParametersFunc", _run, _grad, doc=__doc__)
ema_parameters = EMAParametersFunc.apply
