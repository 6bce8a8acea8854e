"""The generic forward/backward bridge of the fused ops, on CPU tensors."""
import torch

from megalodon_amd.fused_ops._autograd import fused_op


def _make():
    def run(a, b, scale=2.0, flag=True):
        return (a * b * scale, a.detach().sum()), (a, b), scale

    def grad(scale, saved, out_grad, _sum_grad):
        a, b = saved
        return out_grad * b * scale, out_grad * a * scale, None, None

    return fused_op("ScaledProduct", run, grad, non_differentiable=(1,), doc="a * b * scale and sum(a)")


def test_gradients_constants_and_defaults():
    op = _make()
    assert op.__name__ == "ScaledProduct" and issubclass(op, torch.autograd.Function)
    a = torch.randn(5, dtype=torch.float64, requires_grad=True)
    b = torch.randn(5, dtype=torch.float64, requires_grad=True)
    # trailing arguments left at their defaults: two gradients are expected, four are produced
    y, total = op.apply(a, b)
    assert not total.requires_grad
    y.sum().backward()
    assert torch.allclose(a.grad, 2.0 * b.detach()) and torch.allclose(b.grad, 2.0 * a.detach())
    # all arguments given
    a.grad = b.grad = None
    y, _ = op.apply(a, b, 3.0, False)
    y.sum().backward()
    assert torch.allclose(a.grad, 3.0 * b.detach())


def test_saved_none_is_allowed():
    def run(a, maybe):
        return a * 2.0, (a, maybe), None

    def grad(_, saved, g):
        assert saved[1] is None
        return g * 2.0, None

    op = fused_op("Twice", run, grad)
    a = torch.ones(3, requires_grad=True)
    op.apply(a, None).sum().backward()
    assert torch.equal(a.grad, torch.full((3,), 2.0))


def test_linear_layers_on_cpu_tensors_are_plain_linear():
    """`Linear` / `linear_group` off the GPU (or in float32): the values and gradients of
    `F.linear`, layer by layer -- the grouped backward and the own weight-gradient kernel are for
    16-bit tensors on the GPU only."""
    import torch.nn.functional as F
    from megalodon_amd.modules.linear import Linear, linear_group
    torch.manual_seed(0)
    layers = [Linear(12, 7, bias=True).double(), Linear(12, 5, bias=False).double()]
    x = torch.randn(3, 4, 12, dtype=torch.float64, requires_grad=True)
    ys = linear_group(x, layers)
    for y, l in zip(ys, layers):
        assert torch.equal(y, F.linear(x, l.weight, l.bias))
    (ys[0].sum() + 2.0 * ys[1].sum()).backward()
    want = layers[0].weight.detach().sum(0) + 2.0 * layers[1].weight.detach().sum(0)
    assert torch.allclose(x.grad, want.expand_as(x.grad))
    r = torch.randn(3, 4, 5, dtype=torch.float64)
    assert torch.allclose(layers[1](x, residual=r), F.linear(x, layers[1].weight) + r)
