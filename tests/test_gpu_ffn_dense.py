"""Dense gated FFN block (MFMA dispatcher GEMMs + gated-activation kernels) against the CPU oracle:
bf16 tensors at rtol = atol = 1e-2 relative to each tensor's scale."""
from types import SimpleNamespace

import pytest
import torch

from flextrain_amd.ffn_dense import SwiGLUConfig, SwiGLUFFN
from oracle import ffn_dense as o_ffn
from util import gen, randn

pytestmark = pytest.mark.gpu


def _close(a, e, what):
    a, e = a.float().cpu(), e.float()
    scale = max(1.0, float(e.abs().max()))
    torch.testing.assert_close(a, e, rtol=1e-2, atol=1e-2 * scale, msg=lambda m: f"{what}: {m}")


@pytest.mark.parametrize("T,d,f", [(512, 256, 704), (200, 136, 328)])
@pytest.mark.parametrize("activation", ["silu", "gelu_tanh"])
@pytest.mark.parametrize("gdt", [torch.bfloat16, torch.float32])
def test_block_fwd_bwd(dev, T, d, f, activation, gdt):
    g = gen(T + f)
    bf = torch.bfloat16
    h, resid, dy = randn(g, T, d), randn(g, T, d), randn(g, T, d)
    w1, w3, w2 = randn(g, d, f, std=d ** -0.5), randn(g, d, f, std=d ** -0.5), randn(g, f, d, std=f ** -0.5)
    g0 = {"g_1": randn(g, d, f, dtype=gdt), "g_2": randn(g, f, d, dtype=gdt), "g_3": randn(g, d, f, dtype=gdt)}
    out_ref, x1_ref, x3_ref = o_ffn.ffn_fwd(h, w1, w3, w2, resid, activation)
    dx_ref, g1_ref, g2_ref, g3_ref = o_ffn.ffn_bwd(dy, h, x1_ref, x3_ref, w1, w3, w2, g0["g_1"], g0["g_2"], g0["g_3"],
                                                   activation)

    blk = SwiGLUFFN(SwiGLUConfig(d_model=d, expert_dim=f, activation=activation))
    W = {"w_1": w1.to(dev), "w_2": w2.to(dev), "w_3": w3.to(dev)}
    G = {k: v.to(dev) for k, v in g0.items()}
    slot = SimpleNamespace(x1=torch.empty(T, f, dtype=bf, device=dev), x3=torch.empty(T, f, dtype=bf, device=dev), aux={})
    hd, rd = h.to(dev), resid.to(dev)
    out = blk.fwd(hd, W, rd, rd, slot)              # written over the residual, as the engine does
    assert out is rd
    _close(out, out_ref, "out"), _close(slot.x1, x1_ref, "x1"), _close(slot.x3, x3_ref, "x3")

    # the saved activations can be rebuilt bit-identically
    x1_saved = slot.x1.clone()
    slot.x1.zero_()
    blk.fwd_recompute_x1x3(hd, W, slot, recompute_x1=True, recompute_x3=False)
    assert torch.equal(slot.x1, x1_saved)

    dx = blk.bwd(dy.to(dev), W, G, slot)
    assert set(slot.aux) == {"bwd_dx1_up", "bwd_dx3_up"}
    blk.bwd_accumulate_w1_w3_grads(hd, G, slot)
    assert not slot.aux
    _close(dx, dx_ref, "dx"), _close(G["g_1"], g1_ref, "g_1"), _close(G["g_2"], g2_ref, "g_2"), _close(G["g_3"], g3_ref, "g_3")


def test_skip_grads_hands_back_operands(dev):
    g = gen(9)
    T, d, f = 128, 64, 192
    blk = SwiGLUFFN(SwiGLUConfig(d_model=d, expert_dim=f))
    W = {"w_1": randn(g, d, f, std=0.1).to(dev), "w_2": randn(g, f, d, std=0.1).to(dev), "w_3": randn(g, d, f, std=0.1).to(dev)}
    G = {k: torch.zeros_like(W["w_" + k[-1]]) for k in ("g_1", "g_2", "g_3")}
    slot = SimpleNamespace(x1=torch.empty(T, f, dtype=torch.bfloat16, device=dev),
                           x3=torch.empty(T, f, dtype=torch.bfloat16, device=dev), aux={})
    h, dy = randn(g, T, d).to(dev), randn(g, T, d).to(dev)
    blk.fwd(h, W, torch.zeros_like(h), torch.empty_like(h), slot)
    cap = {}
    blk.bwd(dy, W, G, slot, skip_grads=frozenset({"g_2"}), capture_xy=cap)
    blk.bwd_accumulate_w1_w3_grads(h, G, slot, skip_grads=frozenset({"g_1", "g_3"}), capture_xy=cap)
    assert set(cap) == {"g_1", "g_2", "g_3"} and not any(v.any() for v in G.values())
    act, dyc = cap["g_2"]
    assert act.shape == (T, f) and torch.equal(dyc, dy) and cap["g_1"][0] is h


class _MatmulOnly:
    """A dispatcher with the reference's surface only (``matmul``): the blocks must then issue the
    reference's chains of separate calls."""

    def __init__(self):
        from flextrain_amd.matmul_dispatcher import CublasLtDispatcher
        self._d = CublasLtDispatcher()
        self.calls = 0

    def matmul(self, stream_ptr, A, B, C=None, D=None, alpha=1.0, beta=0.0):
        self.calls += 1
        return self._d.matmul(stream_ptr, A, B, C=C, D=D, alpha=alpha, beta=beta)


def test_block_over_a_dispatcher_without_fused_launches(dev):
    g = gen(11)
    T, d, f = 256, 128, 328
    bf = torch.bfloat16
    h, resid, dy = randn(g, T, d), randn(g, T, d), randn(g, T, d)
    w = {"w_1": randn(g, d, f, std=d ** -0.5), "w_3": randn(g, d, f, std=d ** -0.5), "w_2": randn(g, f, d, std=f ** -0.5)}
    results = []
    for disp in (None, _MatmulOnly()):
        blk = SwiGLUFFN(SwiGLUConfig(d_model=d, expert_dim=f, activation="silu"), dispatcher=disp)
        W = {k: v.to(dev) for k, v in w.items()}
        G = {"g_1": torch.zeros(d, f, dtype=bf, device=dev), "g_2": torch.zeros(f, d, dtype=bf, device=dev),
             "g_3": torch.zeros(d, f, dtype=bf, device=dev)}
        slot = SimpleNamespace(x1=torch.empty(T, f, dtype=bf, device=dev), x3=torch.empty(T, f, dtype=bf, device=dev), aux={})
        out = blk.fwd(h.to(dev), W, resid.to(dev), torch.empty(T, d, dtype=bf, device=dev), slot)
        dx = blk.bwd(dy.to(dev), W, G, slot)
        blk.bwd_accumulate_w1_w3_grads(h.to(dev), G, slot)
        results.append((out, dx, G["g_1"], G["g_2"], G["g_3"]))
        if disp is not None:
            assert disp.calls >= 7     # down projection; 4 in bwd (the input gradient as a chain of 2); 2 weight gradients
    for name, a, b in zip(("out", "dx", "g_1", "g_2", "g_3"), *results):
        _close(b, a.float().cpu(), name)
