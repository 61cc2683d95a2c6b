"""Gated activations, SiLU backward, AdamW, embedding backward and RoPE: the kernels' own source run on the
CPU by the host simulation (tests/hostsim) on guard-paged buffers, against the oracle.  Sizes are chosen
for their tails (element counts that are no multiple of a lane's pack or of a workgroup's share) and for
every kernel variant the launch code can pick."""
from __future__ import annotations

import pytest
import torch

from oracle import adamw as o_adam
from oracle import glu as o_glu
from oracle import rope as o_rope
from tests.hostsim import sim

from tests.hostsim.build import needs_host_clang

pytestmark = needs_host_clang

BF, F16, F32 = torch.bfloat16, torch.float16, torch.float32


def _close(a, e, tol=1e-2):
    torch.testing.assert_close(a.float(), e.float(), rtol=tol, atol=tol)


@pytest.mark.parametrize("n", [1, 7, 8, 9, 4095, 4096, 4104, 12345])
@pytest.mark.parametrize("act", [0, 1])
def test_gated_activations(n, act):
    g = torch.Generator().manual_seed(n + act)
    x1, x3, d = (torch.randn(n, generator=g).to(BF) for _ in range(3))
    L = sim.lib()
    out = sim.guard(torch.empty(n, dtype=BF))
    assert L.fx_glu_fwd(sim.p(sim.guard(x1)), sim.p(sim.guard(x3)), sim.p(out), n, 2, 2, act, None) == 0
    fwd, bwd = (o_glu.swiglu_fwd, o_glu.swiglu_bwd) if act == 0 else (o_glu.gelu_tanh_gated_fwd, o_glu.gelu_tanh_gated_bwd)
    _close(out, fwd(x1, x3))
    dx1, dx3, a = (sim.guard(torch.empty(n, dtype=BF)) for _ in range(3))
    assert L.fx_glu_bwd(sim.p(sim.guard(x1)), sim.p(sim.guard(x3)), sim.p(sim.guard(d)), sim.p(dx1), sim.p(dx3), sim.p(a), n, 2,
                        act, None) == 0
    r1, r3, ra = bwd(x1, x3, d)
    _close(dx1, r1, 2e-2), _close(dx3, r3, 2e-2), _close(a, ra)
    dx1b, dx3b = (sim.guard(torch.empty(n, dtype=BF)) for _ in range(2))
    assert L.fx_glu_bwd(sim.p(sim.guard(x1)), sim.p(sim.guard(x3)), sim.p(sim.guard(d)), sim.p(dx1b), sim.p(dx3b), None, n, 2,
                        act, None) == 0
    assert torch.equal(dx1b, dx1) and torch.equal(dx3b, dx3)


@pytest.mark.parametrize("n,dt", [(5, BF), (4096, BF), (4100, BF), (1003, F32), (520, F16)])
def test_silu_backward(n, dt):
    g = torch.Generator().manual_seed(n)
    z, d = torch.randn(n, generator=g).to(dt), torch.randn(n, generator=g).to(dt)
    L = sim.lib()
    out = sim.guard(torch.empty(n, dtype=dt))
    assert L.fx_silu_bwd(sim.p(sim.guard(z)), sim.p(sim.guard(d)), sim.p(out), n, sim.DT[dt], None) == 0
    _close(out, o_glu.silu_bwd(z, d))
    inplace = sim.guard(d)
    assert L.fx_silu_bwd(sim.p(sim.guard(z)), sim.p(inplace), sim.p(inplace), n, sim.DT[dt], None) == 0
    assert torch.equal(inplace, out)


@pytest.mark.parametrize("n", [1, 3, 4, 2047, 2048, 2052, 10007])
@pytest.mark.parametrize("pdt,gdt,sdt", [(F32, BF, F32), (BF, BF, BF), (F32, F32, F32), (BF, BF, F32)])
def test_adamw(n, pdt, gdt, sdt):
    g = torch.Generator().manual_seed(n)
    p = (torch.randn(n, generator=g) * 0.02).to(pdt)
    gr = (torch.randn(n, generator=g) * 1e-3).to(gdt)
    m = (torch.randn(n, generator=g) * 1e-4).to(sdt)
    v = (torch.rand(n, generator=g) * 1e-6).to(sdt)
    hp = dict(lr=3e-3, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
    step = 3
    L = sim.lib()
    gp, gm, gv, copy = sim.guard(p), sim.guard(m), sim.guard(v), sim.guard(torch.empty(n, dtype=BF))
    assert L.fx_adamw_step(sim.p(gp), sim.p(sim.guard(gr)), sim.p(gm), sim.p(gv), sim.p(copy), n, sim.DT[pdt], sim.DT[gdt], sim.DT[sdt],
                           hp["lr"], hp["beta1"], hp["beta2"], hp["eps"], hp["weight_decay"], 1 - hp["beta1"] ** step,
                           1 - hp["beta2"] ** step, None) == 0
    rp, rm, rv, rc = o_adam.adamw_step(p, gr, m, v, step=step, **hp)
    tol = 1e-2 if pdt == BF else 1e-5
    torch.testing.assert_close(gp.float(), rp.float(), rtol=tol, atol=tol * 1e-2)
    torch.testing.assert_close(gm.float(), rm.float(), rtol=1e-2 if sdt == BF else 1e-5, atol=1e-7)
    torch.testing.assert_close(gv.float(), rv.float(), rtol=1e-2 if sdt == BF else 1e-5, atol=1e-9)
    torch.testing.assert_close(copy.float(), rc.float(), rtol=1e-2, atol=1e-4)
    flag = sim.guard(torch.zeros(1, dtype=torch.int32))
    assert L.fx_nonfinite_flag(sim.p(gp), n, sim.DT[pdt], sim.p(flag), None) == 0 and int(flag) == 0
    gp[n // 2] = float("inf")
    assert L.fx_nonfinite_flag(sim.p(gp), n, sim.DT[pdt], sim.p(flag), None) == 0 and int(flag) == 1


@pytest.mark.parametrize("T,D,V,idt", [(37, 64, 11, torch.int32), (200, 40, 300, torch.int64), (5, 7, 3, torch.int32)])
def test_embedding_backward(T, D, V, idt):
    g = torch.Generator().manual_seed(T)
    go = torch.randn(T, D, generator=g).to(BF)
    tok = torch.randint(0, V, (T,), generator=g)
    gw = torch.randn(V, D, generator=g)
    order = torch.argsort(tok, stable=True)
    L = sim.lib()
    out = sim.guard(gw)
    assert L.fx_embedding_bwd(sim.p(sim.guard(go)), sim.p(sim.guard(order.to(idt))), sim.p(sim.guard(tok[order].to(idt))),
                              int(idt == torch.int64), sim.p(out), T, D, V, D, 1, D, 1, 0.5, 2, 0, None) == 0
    torch.testing.assert_close(out, o_glu.embedding_bwd(go, tok, gw, scale=0.5), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("T,Hq,Hk,D,rot", [(9, 32, 8, 128, 128), (5, 4, 4, 64, 64), (7, 3, 1, 64, 32), (130, 2, 0, 128, 128),
                                          (6, 5, 2, 256, 64), (3, 40, 8, 128, 128)])
@pytest.mark.parametrize("backward", [0, 1])
def test_rope(T, Hq, Hk, D, rot, backward):
    g = torch.Generator().manual_seed(T * D + Hq)
    q = torch.randn(T, Hq, D, generator=g).to(BF)
    k = torch.randn(T, max(Hk, 1), D, generator=g).to(BF)
    pos = torch.randint(0, 5000, (T, 1), generator=g, dtype=torch.int32)
    inv = o_rope.vanilla_inv_freq(rot, 500000.0)
    L = sim.lib()
    gq, gk = sim.guard(q), sim.guard(k)
    strides = lambda t: sim.guard(torch.tensor(t.stride(), dtype=torch.int64))
    assert L.fx_rope(sim.p(gq), sim.p(gk) if Hk else None, sim.p(sim.guard(pos)), 1, sim.p(sim.guard(inv)), 1, T, Hq, Hk, D, rot,
                     sim.pi64(strides(gq)), sim.pi64(strides(gk)) if Hk else None, 2, backward, None) == 0
    _close(gq, o_rope.rope(q, pos, inv, backward=bool(backward), rot_dim=rot))
    if Hk:
        _close(gk, o_rope.rope(k, pos, inv, backward=bool(backward), rot_dim=rot))


def test_rope_on_strided_views_of_a_fused_projection():
    """q and k as column slices of one (T, (Hq + 2 Hk) D) projection output: token stride larger than the rows."""
    T, Hq, Hk, D = 11, 4, 2, 64
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn(T, (Hq + 2 * Hk) * D, generator=g).to(BF)
    pos = torch.arange(T, dtype=torch.int32)
    inv = o_rope.vanilla_inv_freq(D, 10000.0)
    buf = sim.guard(qkv)
    q = buf[:, :Hq * D].view(T, Hq, D)
    k = buf[:, Hq * D:(Hq + Hk) * D].view(T, Hk, D)
    L = sim.lib()
    st = lambda t: sim.guard(torch.tensor(t.stride(), dtype=torch.int64))
    assert L.fx_rope(sim.p(q), sim.p(k), sim.p(sim.guard(pos)), 1, sim.p(sim.guard(inv)), 1, T, Hq, Hk, D, D, sim.pi64(st(q)), sim.pi64(st(k)),
                     2, 0, None) == 0
    ref = qkv.clone()
    ref[:, :Hq * D] = o_rope.rope(qkv[:, :Hq * D].view(T, Hq, D), pos, inv).reshape(T, -1)
    ref[:, Hq * D:(Hq + Hk) * D] = o_rope.rope(qkv[:, Hq * D:(Hq + Hk) * D].view(T, Hk, D), pos, inv).reshape(T, -1)
    _close(buf, ref)
    assert torch.equal(buf[:, (Hq + Hk) * D:], qkv[:, (Hq + Hk) * D:])       # v is untouched
