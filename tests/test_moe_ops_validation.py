"""Argument checks of the MoE op wrappers, on the CPU: which mistakes are refused and with which exception
type (the reference's: ValueError for device / shape / contiguity, TypeError for dtypes), and that a
well-formed call reaches the library with the pointers and sizes of its operands.  The device check is
switched off and the library replaced by a recorder, so CPU tensors serve."""
from __future__ import annotations

import pytest
import torch

from flextrain_amd.ops import moe

BF = torch.bfloat16


class _Recorder:
    def __init__(self):
        self.calls = []

    def __getattr__(self, name):
        def call(*args):
            self.calls.append((name, args))
            return 64 if name.endswith("_ws_bytes") else 0
        return call


@pytest.fixture
def rec(monkeypatch):
    r = _Recorder()
    monkeypatch.setattr(moe, "_on_gpu", lambda **kw: None)
    monkeypatch.setattr(moe, "lib", lambda: r)
    monkeypatch.setattr(moe, "stream_ptr", lambda dev: 0)
    return r


def test_device_check_names_the_argument():
    with pytest.raises(ValueError, match="gate_logits must be a CUDA tensor"):
        moe.flextrain_fused_topk_softmax(torch.zeros(4, 8, dtype=BF), 2)
    with pytest.raises(ValueError, match="indices must be a CUDA tensor"):
        moe._on_gpu(x=None, indices=torch.zeros(2, 2, dtype=torch.int32))


def test_topk(rec):
    logits = torch.zeros(16, 8, dtype=BF)
    w, ids = moe.flextrain_fused_topk_softmax(logits, 2)
    assert w.shape == (16, 2) and w.dtype == BF and ids.dtype == torch.int32
    name, args = rec.calls[-1]
    assert name == "fx_topk_softmax" and args[0] == logits.data_ptr() and args[3:6] == (16, 8, 2)
    for bad in (dict(top_k=9), dict(mode="nearest"), dict(topk_ids_out=torch.zeros(16, 3, dtype=torch.int32)),
                dict(topk_weights_out=torch.zeros(2, 16, dtype=BF).t())):
        kw = dict(dict(top_k=2), **bad)
        with pytest.raises(ValueError):
            moe.flextrain_fused_topk_softmax(logits, **kw)
    with pytest.raises(TypeError):
        moe.flextrain_fused_topk_softmax(logits, 2, topk_ids_out=torch.zeros(16, 2, dtype=torch.int64))
    with pytest.raises(ValueError):
        moe.flextrain_fused_topk_softmax(logits.view(2, 8, 8), 2)
    with pytest.raises(ValueError):
        moe.flextrain_fused_topk_softmax(torch.zeros(8, 16, dtype=BF).t(), 2)


def test_sort_and_counts(rec):
    ids = torch.zeros(10, 4, dtype=torch.int32)
    mapping, counts = moe.flextrain_moe_sort(ids, 16)
    assert mapping.shape == ids.shape and mapping.dtype == torch.int32 and counts.shape == (16,)
    assert [c[0] for c in rec.calls] == ["fx_moe_sort_ws_bytes", "fx_moe_sort"]
    assert rec.calls[-1][1][2:4] == (40, 16)
    with pytest.raises(ValueError):
        moe.flextrain_moe_sort(ids, 16, indices=torch.zeros(10, 5, dtype=torch.int32))
    with pytest.raises(ValueError):
        moe.flextrain_moe_sort(ids, 16, expert_counts_pinned=torch.zeros(16, dtype=torch.int32))     # not pinned
    with pytest.raises(TypeError):
        moe.flextrain_moe_sort(ids.float(), 16)
    with pytest.raises(ValueError):
        moe.flextrain_copy_expert_counts(torch.zeros(16, dtype=torch.int32), torch.zeros(16, dtype=torch.int32))


def test_scatter_gather(rec):
    T, K, D = 6, 2, 16
    x = torch.zeros(T, D, dtype=BF)
    idx = torch.zeros(T, K, dtype=torch.int32)
    out = moe.flextrain_moe_scatter(x, idx)
    assert out.shape == (T * K, D) and rec.calls[-1][0] == "fx_moe_scatter"
    for bad in (dict(indices=idx[:-1]), dict(indices=idx.view(-1)), dict(scales=torch.zeros(T, dtype=BF)),
                dict(out=torch.zeros(T * K, D + 8, dtype=BF)), dict(out=torch.zeros(T * K, D)),
                dict(x=torch.zeros(D, T, dtype=BF).t())):
        kw = dict(dict(x=x, indices=idx), **bad)
        with pytest.raises(ValueError):
            moe.flextrain_moe_scatter(**kw)
    y = torch.zeros(T * K, D, dtype=BF)
    got = moe.flextrain_moe_gather(y, idx, weights=torch.zeros(T, K, dtype=BF), residual=torch.zeros(T, D, dtype=torch.float32))
    assert got.shape == (T, D) and got.dtype == torch.float32          # the residual's dtype
    assert rec.calls[-1][0] == "fx_moe_gather"
    for bad in (dict(expert_out=y[:-1]), dict(weights=torch.zeros(T * K, dtype=BF)), dict(residual=torch.zeros(T, D + 1)),
                dict(out=torch.zeros(T + 1, D, dtype=BF)), dict(indices=idx.view(-1)), dict(expert_out=y.view(-1))):
        kw = dict(dict(expert_out=y, indices=idx), **bad)
        with pytest.raises(ValueError):
            moe.flextrain_moe_gather(**kw)
    w = torch.zeros(T, K, dtype=BF)
    assert moe.flextrain_moe_scatter_routing_weights(w, idx).shape == (T * K,)
    with pytest.raises(ValueError):
        moe.flextrain_moe_scatter_routing_weights(w[:, :1], idx)
    with pytest.raises(ValueError):
        moe.flextrain_moe_scatter_routing_weights(w, idx, out=torch.zeros(T * K + 1, dtype=BF))
    with pytest.raises(ValueError):
        moe.flextrain_moe_row_sources(idx, out=torch.zeros(T * K, dtype=torch.int64))


def test_expert_activation(rec):
    T, F = 8, 16
    x = torch.zeros(T, 2 * F, dtype=BF)
    assert moe.flextrain_swiglu_moe_fwd(x).shape == (T, F)
    assert moe.flextrain_swiglu_moe_fwd(x, w=torch.zeros(T, 1, dtype=BF)).shape == (T, F)
    for bad in (dict(x=torch.zeros(T, 2 * F + 1, dtype=BF)), dict(out=torch.zeros(T, F + 1, dtype=BF)),
                dict(w=torch.zeros(T + 1, dtype=BF)), dict(x=torch.zeros(2 * F, T, dtype=BF).t())):
        kw = dict(dict(x=x), **bad)
        with pytest.raises(ValueError):
            moe.flextrain_swiglu_moe_fwd(**kw)
    dout, w = torch.zeros(T, F, dtype=BF), torch.zeros(T, 1, dtype=BF)
    dx, dw = moe.flextrain_swiglu_moe_bwd(dout, x, w)
    assert dx.shape == x.shape and dw.shape == (T,) and dw.dtype == torch.float32
    assert rec.calls[-1][0] == "fx_swiglu_moe_bwd" and rec.calls[-1][1][-2] == 0
    moe.flextrain_swiglu_moe_bwd_prescaled(dout, x, w, fwd_act=torch.zeros(T, F, dtype=BF))
    assert rec.calls[-1][1][-2] == 1                                   # the prescaled flag
    for bad in (dict(x=x[:-1]), dict(x=torch.zeros(T, 2 * F + 2, dtype=BF)), dict(w=torch.zeros(T - 1, dtype=BF)),
                dict(dx=torch.zeros(T, F, dtype=BF)), dict(dw=torch.zeros(T + 1)), dict(fwd_act=torch.zeros(T, 2 * F, dtype=BF))):
        kw = dict(dict(dout=dout, x=x, w=w), **bad)
        with pytest.raises(ValueError):
            moe.flextrain_swiglu_moe_bwd(**kw)
    with pytest.raises(TypeError):
        moe.flextrain_swiglu_moe_bwd(dout.float(), x, w)


def test_router_backward(rec):
    T, K, E = 8, 2, 16
    probs, dprobs = torch.zeros(T, K, dtype=BF), torch.zeros(T * K, 1, dtype=BF)
    idx, chosen = torch.zeros(T, K, dtype=torch.int32), torch.zeros(T, K, dtype=torch.int32)
    dl = moe.flextrain_moe_router_gate_bwd(probs, dprobs, idx, chosen, num_experts=E)
    assert dl.shape == (T, E) and rec.calls[-1][0] == "fx_router_gate_bwd"
    logits = torch.zeros(T, E, dtype=BF)
    moe.flextrain_moe_router_gate_bwd(probs, dprobs, idx, chosen, dlogits=dl, mode="softmax_then_topk", logits=logits)
    for bad in (dict(), dict(num_experts=E, dprobs=dprobs[:-1]), dict(num_experts=E, indices=idx[:, :1]),
                dict(num_experts=E, chosen_experts=chosen[:-1]), dict(dlogits=torch.zeros(T + 1, E, dtype=BF)),
                dict(dlogits=dl, mode="softmax_then_topk"), dict(dlogits=dl, mode="softmax_then_topk", logits=logits[:, :-1]),
                dict(num_experts=E, mode="nearest")):
        kw = dict(dict(probs=probs, dprobs=dprobs, indices=idx, chosen_experts=chosen), **bad)
        with pytest.raises(ValueError):
            moe.flextrain_moe_router_gate_bwd(**kw)
    with pytest.raises(TypeError):
        moe.flextrain_moe_router_gate_bwd(probs, dprobs, idx, chosen, dlogits=dl.float())
    counts = torch.zeros(E, dtype=torch.int32)
    assert moe.flextrain_load_balance_bwd(logits, counts, E, K).shape == (T, E)
    args = rec.calls[-1][1]
    assert rec.calls[-1][0] == "fx_load_balance_bwd" and abs(args[6] - 0.01 * E / T) < 1e-9     # tokens_per_step defaults to T
    for bad in (dict(num_experts=E + 1), dict(expert_counts=counts[:-1]), dict(dlogits=torch.zeros(T, E + 1, dtype=BF)),
                dict(logits=torch.zeros(E, T, dtype=BF).t())):
        kw = dict(dict(logits=logits, expert_counts=counts, num_experts=E, top_k=K), **bad)
        with pytest.raises(ValueError):
            moe.flextrain_load_balance_bwd(**kw)
