"""`attention_softmax(x, dropout, use_causal_mask, training) -> y`: row softmax
of attention scores with the bottom-right aligned causal mask and DropKey, as
the op of megalodon/modules/fused_ops/attention/softmax.py:9-35.  Backward
needs y only: a dropped key has probability 0 and so no gradient."""
from ... import extension as ops
from .._autograd import fused_op


def _run(x, dropout=0.0, use_causal_mask=True, training=True):
    y = ops.attention_softmax_fwd(x, dropout if training else 0.0, use_causal_mask)
    return y, (y,), use_causal_mask


def _grad(use_causal_mask, saved, y_grad):
    return ops.attention_softmax_bwd(y_grad, saved[0], use_causal_mask), None, None, None


AttentionSoftmaxFunc = fused_op("AttentionSoftmaxFunc", _run, _grad, doc=__doc__)
attention_softmax = AttentionSoftmaxFunc.apply
