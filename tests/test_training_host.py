"""Host-side pieces of the training path that need no GPU."""
import torch

from landmarksystem_amd.anchor_decoder import _TallLinear, _mlp


def test_tall_linear_equals_nn_linear_in_value_and_gradients():
    """The slab-wise weight gradient (whole slabs through one batched product, the tail through a plain one) against
    autograd through torch.nn.functional.linear, in float64: rows = 2 slabs + a tail, then fewer rows than a slab."""
    g = torch.Generator().manual_seed(0)
    for rows in (2 * _TallLinear.SLAB + 37, 100, _TallLinear.SLAB):
        x = torch.randn(rows, 35, generator=g, dtype=torch.float64, requires_grad=True)
        w = torch.randn(32, 35, generator=g, dtype=torch.float64, requires_grad=True)
        b = torch.randn(32, generator=g, dtype=torch.float64, requires_grad=True)
        cot = torch.randn(rows, 32, generator=g, dtype=torch.float64)
        got = _TallLinear.apply(x, w, b)
        want = torch.nn.functional.linear(x, w, b)
        assert torch.allclose(got, want, rtol=0, atol=1e-12)
        grads = torch.autograd.grad((got * cot).sum(), (x, w, b))
        ref = torch.autograd.grad((want * cot).sum(), (x, w, b))
        for a, r in zip(grads, ref):
            assert torch.allclose(a, r, rtol=1e-12, atol=1e-10)


def test_mlp_helper_follows_the_sequential_module():
    seq = torch.nn.Sequential(torch.nn.Linear(35, 32), torch.nn.ReLU(True), torch.nn.Linear(32, 10), torch.nn.Tanh()).double()
    x = torch.randn(50, 35, dtype=torch.float64)
    assert torch.allclose(_mlp(seq, x), seq(x.clone()), rtol=0, atol=1e-12)
    # a view whose rows are not contiguous
    wide = torch.randn(50, 70, dtype=torch.float64)
    assert torch.allclose(_mlp(seq, wide[:, ::2]), seq(wide[:, ::2].clone()), rtol=0, atol=1e-12)
