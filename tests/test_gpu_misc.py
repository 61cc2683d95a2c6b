"""SiLU backward and embedding backward against the CPU oracle, plus the module-level objects of
the reference's ``flextrain.ops`` surface (dispatchers, pinned-memory helpers)."""
import pytest
import torch
import torch.nn.functional as F

from flextrain_amd import ops
from oracle import glu as o_glu
from util import close, gen, randn

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape", [(32768, 8192), (1000, 77), (5,), (3, 8)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_silu_bwd(dev, shape, dtype):
    g = gen(sum(shape))
    if shape == (32768, 8192) and dtype == torch.float32:
        pytest.skip("the large shape is covered in bf16")
    z, dout = randn(g, *shape, dtype=dtype, std=2.0), randn(g, *shape, dtype=dtype)
    ref = o_glu.silu_bwd(z, dout)
    # the oracle against autograd on a slice
    zs = z.flatten()[:4096].float().requires_grad_()
    (gz,) = torch.autograd.grad((F.silu(zs) * dout.flatten()[:4096].float()).sum(), zs)
    torch.testing.assert_close(ref.flatten()[:4096].float(), gz.to(dtype).float(), rtol=1e-2, atol=1e-2)
    zd, dd = z.to(dev), dout.to(dev)
    din = ops.flextrain_silu_bwd(zd, dd)
    close(din, ref, rtol=1e-2 if dtype == torch.bfloat16 else 1e-5, atol=1e-2 if dtype == torch.bfloat16 else 1e-6)
    # in place over dout
    out = ops.flextrain_silu_bwd(zd, dd, din=dd)
    assert out is dd and torch.equal(dd, din)
    with pytest.raises(AssertionError):
        ops.flextrain_silu_bwd(zd, dd.flatten()[:-1])


@pytest.mark.parametrize("T,D,V", [(4096, 1024, 32000), (300, 72, 50), (17, 5, 9)])
@pytest.mark.parametrize("gdt,wdt,idt", [(torch.bfloat16, torch.bfloat16, torch.int64), (torch.bfloat16, torch.float32, torch.int32)])
def test_embedding_bwd(dev, T, D, V, gdt, wdt, idt):
    g = gen(T + D)
    go = randn(g, T, D, dtype=gdt)
    idx = torch.randint(0, V, (T,), generator=g).to(idt)
    idx[: T // 4] = 3                               # a heavily repeated token
    gw0 = randn(g, V, D, dtype=wdt, std=0.5)
    ref = o_glu.embedding_bwd(go, idx, gw0, scale=0.5)
    # oracle against autograd through F.embedding
    w = torch.zeros(V, D, requires_grad=True)
    (gw_auto,) = torch.autograd.grad((F.embedding(idx.long(), w) * 0.5 * go.float()).sum(), w)
    torch.testing.assert_close(ref.float(), (gw0.float() + gw_auto).to(wdt).float(), rtol=1e-2, atol=1e-2)
    gw = gw0.to(dev).clone()
    out = ops.flextrain_embedding_bwd(go.to(dev), idx.to(dev), gw, scale=0.5)
    assert out is gw
    tol = 1e-2 if wdt == torch.bfloat16 else 1e-4
    close(gw, ref, rtol=tol, atol=tol * max(1.0, float(ref.float().abs().max())))
    untouched = torch.ones(V, dtype=torch.bool)
    untouched[idx.long()] = False
    assert torch.equal(gw.cpu()[untouched], gw0[untouched])
    # reproducible: the same call gives the same bits
    gw2 = gw0.to(dev).clone()
    ops.flextrain_embedding_bwd(go.to(dev), idx.to(dev), gw2, scale=0.5)
    assert torch.equal(gw, gw2)


def test_ops_surface_objects(dev):
    from flextrain_amd.matmul_dispatcher import CublasLtDispatcher
    assert isinstance(ops.dispatcher, CublasLtDispatcher) and isinstance(ops.dispatcher_secondary, CublasLtDispatcher)
    assert ops.dispatcher is ops.dispatcher and ops.dispatcher is not ops.dispatcher_secondary
    t = ops.pin_tensor(torch.arange(16, dtype=torch.float32))
    assert t.is_pinned()
    ops.destroy_pinned_tensor(t)
    with pytest.raises(AttributeError):
        ops.no_such_thing
