"""HIP gated activations against the CPU oracle (bf16 rtol = atol = 1e-2) and
the reference's own unit-test shapes (tests/test_gelu_tanh_gated_kernel.py:47-104)."""
import pytest
import torch

from flextrain_amd import ops
from oracle import glu as o_glu
from util import close, gen, randn

pytestmark = pytest.mark.gpu

FAMILIES = {
    "swiglu": (ops.flextrain_swiglu_fwd, ops.flextrain_swiglu_bwd, o_glu.swiglu_fwd, o_glu.swiglu_bwd),
    "gelu": (ops.flextrain_gelu_tanh_gated_fwd, ops.flextrain_gelu_tanh_gated_bwd,
             o_glu.gelu_tanh_gated_fwd, o_glu.gelu_tanh_gated_bwd),
}
SHAPES = [(64, 256), (32, 1152), (8, 6912), (1024, 14336), (3, 5), (1, 1), (17, 4099)]


@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fwd_bwd(dev, family, shape, dtype):
    fwd, bwd, ofwd, obwd = FAMILIES[family]
    g = gen(7 if family == "gelu" else 11)
    x1, x3, d = (randn(g, *shape, dtype=dtype) for _ in range(3))
    tol = 1e-2 if dtype == torch.bfloat16 else 2e-5
    out = fwd(x1.to(dev), x3.to(dev))
    close(out, ofwd(x1, x3), rtol=tol, atol=tol, what="out")
    dx1, dx3, act = bwd(x1.to(dev), x3.to(dev), d.to(dev), store_activations=True)
    r1, r3, ract = obwd(x1, x3, d)
    close(dx1, r1, rtol=tol, atol=tol, what="dx1")
    close(dx3, r3, rtol=tol, atol=tol, what="dx3")
    close(act, ract, rtol=tol, atol=tol, what="act")
    assert torch.equal(act, out), "stored activation must equal the forward output"
    two = bwd(x1.to(dev), x3.to(dev), d.to(dev))
    assert len(two) == 2 and torch.equal(two[0], dx1) and torch.equal(two[1], dx3)


def test_reference_unit_test_metrics(dev):
    """cos >= 0.9995 and rel-L2 <= 1e-2 against fp32 autograd
    (tests/test_gelu_tanh_gated_kernel.py:36-38)."""
    g = gen(7)
    x1, x3, d = (randn(g, 32, 1152) for _ in range(3))
    a = x1.float().requires_grad_()
    b = x3.float().requires_grad_()
    out = torch.nn.functional.gelu(a, approximate="tanh") * b
    g1, g3 = torch.autograd.grad(out, (a, b), d.float())
    dx1, dx3 = ops.flextrain_gelu_tanh_gated_bwd(x1.to(dev), x3.to(dev), d.to(dev))
    for got, ref in ((dx1, g1), (dx3, g3)):
        got = got.float().cpu().flatten()
        ref = ref.flatten()
        assert torch.nn.functional.cosine_similarity(got, ref, dim=0) >= 0.9995
        assert (got - ref).norm() / ref.norm() <= 1e-2


def test_full_size_swiglu(dev):
    """gate/up [8192,14336]: compare a row band against the oracle, and the
    whole tensor through linearity in x3 and dout (size-independent)."""
    g = gen(1001)
    T, F = 8192, 14336
    x1 = randn(g, T, F).to(dev)
    x3 = randn(g, T, F).to(dev)
    d = randn(g, T, F).to(dev)
    out = ops.flextrain_swiglu_fwd(x1, x3)
    dx1, dx3, act = ops.flextrain_swiglu_bwd(x1, x3, d, store_activations=True)
    rows = slice(4000, 4064)
    c = lambda t: t[rows].cpu()
    close(out[rows], o_glu.swiglu_fwd(c(x1), c(x3)))
    r1, r3, _ = o_glu.swiglu_bwd(c(x1), c(x3), c(d))
    close(dx1[rows], r1)
    close(dx3[rows], r3)
    assert torch.equal(act, out)
    # out is linear in x3: f(x1, 2*x3) == 2*f(x1, x3) exactly in bf16 (power of two)
    assert torch.equal(ops.flextrain_swiglu_fwd(x1, x3 * 2), out * 2)
    # dx3 does not depend on x3; dx1 is linear in dout
    dx1b, dx3b = ops.flextrain_swiglu_bwd(x1, x3 * 2, d * 2)
    assert torch.equal(dx3b, dx3 * 2)


def test_out_buffers_noncontiguous_inputs(dev):
    g = gen(3)
    x1, x3, d = (randn(g, 64, 96) for _ in range(3))
    out = torch.empty(64, 96, dtype=torch.bfloat16, device=dev)
    r = ops.flextrain_swiglu_fwd(x1.to(dev), x3.to(dev), out=out)
    assert r is out
    x1t = x1.t().contiguous().to(dev).t()  # same values, non-contiguous
    assert not x1t.is_contiguous()
    assert torch.equal(ops.flextrain_swiglu_fwd(x1t, x3.to(dev)), out)
    dx1 = torch.empty_like(out)
    dx3 = torch.empty_like(out)
    a, b = ops.flextrain_swiglu_bwd(x1.to(dev), x3.to(dev), d.to(dev), dx1=dx1, dx3=dx3)
    assert a is dx1 and b is dx3
    e = torch.empty(0, 8, dtype=torch.bfloat16, device=dev)
    assert ops.flextrain_swiglu_fwd(e, e).shape == (0, 8)
