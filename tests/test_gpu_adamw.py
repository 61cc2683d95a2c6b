"""HIP AdamW against the CPU oracle: fp32 parameters and optimizer state at
rtol 1e-4; the absolute floors (p 1e-9, m 1e-8, v 1e-12) are 1e-4 of each
quantity's typical magnitude here (p ~2e-2, m ~1e-4, v ~5e-8) and only matter
where beta*m and (1-beta)*g cancel;
bf16 state at rtol = atol = 1e-2."""
import pytest
import torch

from flextrain_amd import ops
from oracle import adamw as o_adamw
from util import close, gen, randn

pytestmark = pytest.mark.gpu

HP = dict(lr=3e-5, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)


@pytest.mark.parametrize("n", [1, 7, 8, 4096, 1_000_003])
def test_fp32_master_four_steps(dev, n):
    g = gen(1003)
    p = randn(g, n, dtype=torch.float32, std=0.02)
    m, v = torch.zeros(n), torch.zeros(n)
    pd, md, vd = p.to(dev), m.to(dev), v.to(dev)
    pb = torch.empty(n, dtype=torch.bfloat16, device=dev)
    for step in range(1, 5):
        grad = randn(g, n, std=1e-3)
        p, m, v, pbf = o_adamw.adamw_step(p, grad, m, v, step=step, **HP)
        rc = ops.flextrain_adamw_step(pd, grad.to(dev), md, vd, step=step, params_bf16_out=pb, **HP)
        assert rc == 0
        close(pd, p, rtol=1e-4, atol=1e-9, what=f"p step {step}")
        close(md, m, rtol=1e-4, atol=1e-8, what=f"m step {step}")
        close(vd, v, rtol=1e-4, atol=1e-12, what=f"v step {step}")
        close(pb, pbf, rtol=1e-2, atol=1e-2, what="bf16 copy")
        assert torch.equal(pb, pd.to(torch.bfloat16))


def test_compute_dtype_slot_bf16_everything(dev):
    # the engine's default: params and state in bf16 (flextrain/optim/adamw.py:110-120)
    g = gen(5)
    n = 50000
    p, grad = randn(g, n, std=0.02), randn(g, n, std=1e-3)
    m, v = randn(g, n, std=1e-4), randn(g, n, std=1e-4).abs()
    rp, rm, rv, _ = o_adamw.adamw_step(p, grad, m, v, step=3, **HP)
    pd, md, vd = p.to(dev), m.to(dev), v.to(dev)
    assert ops.flextrain_adamw_step(pd, grad.to(dev), md, vd, step=3, **HP) == 0
    close(pd, rp), close(md, rm), close(vd, rv)


def test_check_error_returns_minus_one_and_leaves_state(dev):
    n = 1000
    p = torch.ones(n, device=dev)
    m = torch.zeros(n, device=dev)
    v = torch.zeros(n, device=dev)
    for bad in (float("nan"), float("inf"), float("-inf")):
        grad = torch.zeros(n, device=dev, dtype=torch.bfloat16)
        grad[n // 2] = bad
        assert ops.flextrain_adamw_step(p, grad, m, v, check_error=True) == -1
        assert torch.equal(p, torch.ones_like(p)) and not m.any() and not v.any()
    good = torch.zeros(n, device=dev, dtype=torch.bfloat16)
    assert ops.flextrain_adamw_step(p, good, m, v, check_error=True) == 0


def test_errors(dev):
    with pytest.raises(ValueError):
        ops.flextrain_adamw_step(torch.ones(4), torch.ones(4), torch.ones(4), torch.ones(4))
    e = torch.zeros(0, device=dev)
    assert ops.flextrain_adamw_step(e, e, e, e) == 0


def test_full_size_offloaded_layer_chunk(dev):
    """218,112,000 parameters (one Llama-3.1-8B decoder layer), fp32 master weights and moments, bf16
    gradients, three prior steps, the measured step is step 4, bf16 copy of the new weights; against
    the CPU oracle on every element (fp32 state: rtol 1e-4, absolute floors as in the test above)."""
    n = 218_112_000
    g = gen(1003)
    p = torch.empty(n).normal_(0, 0.02, generator=g)
    m = torch.zeros(n)
    v = torch.zeros(n)
    pd, md, vd = p.to(dev), m.to(dev), v.to(dev)
    pb = torch.empty(n, dtype=torch.bfloat16, device=dev)
    for step in range(1, 5):
        gr = torch.empty(n).normal_(0, 1e-3, generator=g).to(torch.bfloat16)
        p, m, v, pbf = o_adamw.adamw_step(p, gr, m, v, step=step, **HP)
        assert ops.flextrain_adamw_step(pd, gr.to(dev), md, vd, step=step, params_bf16_out=pb, **HP) == 0
    torch.testing.assert_close(pd.cpu(), p, rtol=1e-4, atol=1e-9)
    torch.testing.assert_close(md.cpu(), m, rtol=1e-4, atol=1e-8)
    torch.testing.assert_close(vd.cpu(), v, rtol=1e-4, atol=1e-12)
    assert torch.equal(pb.cpu(), pd.to(torch.bfloat16).cpu())
