"""The per-layer parameter / gradient / optimizer-state rings and the streamed optimizer step
over them (reference: BufferManager accessors flextrain/engine/buffers.py:981-1034, :1088-1297;
pipeline of ActiveModel.step flextrain/engine/active_model.py:486-655).  The pipelined,
three-stream schedule must leave the pinned host tables bit-equal to a synchronous run of
the same step, and equal to the CPU oracle's AdamW within fp32 rtol 1e-4."""
import pytest
import torch

from flextrain_amd.layer_ring import LayerRingBuffers, RingParamSpec, RingTensor, ring_optimizer_step
from flextrain_amd.optim import AdamW, AdamWHyperparams, state_key
from flextrain_amd.streams import EventBook, StreamBundle
from oracle import adamw as o_adamw
from util import gen

pytestmark = pytest.mark.gpu

HP = dict(lr=3e-5, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)


def _specs(n_layers):
    """Heterogeneous layers: shapes differ from layer to layer, one tensor is frozen, some
    element counts are not multiples of the packing granule."""
    specs = []
    for i in range(n_layers):
        d = 256 + 64 * (i % 3)
        specs.append(RingParamSpec((RingTensor("w_q", (d, 512)), RingTensor("w_frozen_emb", (100 + i, 33), True),
                                    RingTensor("w_o", (512, d + 1)), RingTensor("attn_norm", (d + 3,)))))
    return specs


def _fill(buf, seed):
    g = gen(seed)
    for lid in range(len(buf.layer_param_specs)):
        for t in buf.host_params[lid].values():
            t.normal_(0, 0.02, generator=g)
        for t in buf.host_grads[lid].values():
            t.copy_(torch.empty(t.shape).normal_(0, 1e-3, generator=g))
        for k, t in buf.host_opt[lid].items():
            t.normal_(0, 1e-3, generator=g)
            if k.startswith("o_adam_v"):
                t.square_()


def _snapshot(buf):
    return [dict(p={k: v.clone() for k, v in buf.host_params[l].items()},
                 g={k: v.clone() for k, v in buf.host_grads[l].items()},
                 o={k: v.clone() for k, v in buf.host_opt[l].items()}) for l in range(len(buf.layer_param_specs))]


def _make(dev, n_layers, n_p, n_g, seed):
    specs = _specs(n_layers)
    buf = LayerRingBuffers(specs, device=dev, n_param_slots=n_p, n_grad_slots=n_g, act_ring_bytes=16 << 20)
    _fill(buf, seed)
    return specs, buf


def test_slot_views_and_single_layer_round_trip(dev):
    specs, buf = _make(dev, 3, 2, 2, 1)
    sb = StreamBundle.create(dev)
    p_views = buf.gpu_param_slot(1, specs[2])
    assert set(p_views) == {"w_q", "w_frozen_emb", "w_o", "attn_norm"} and p_views["w_o"].shape == (512, 385)
    assert set(buf.gpu_grad_slot(0, specs[0])) == {"g_q", "g_o", "g_attn_norm"}
    with pytest.raises(RuntimeError):
        buf.gpu_opt_slot(0, 0)                                   # only valid in optimizer-state mode
    with pytest.raises(RuntimeError):
        buf.fetch_layer_params(0, 0)                             # default stream: refused
    buf.swap_to_optimizer_state(2)
    assert set(buf.gpu_opt_slot(1, 2)) == {state_key(s, n) for s in ("o_adam_m", "o_adam_v")
                                           for n in ("w_q", "w_o", "attn_norm")}
    with pytest.raises(RuntimeError):
        buf.swap_to_optimizer_state(10 ** 6)
    # frozen regions share a base across layers: fetching layer 0's trainable part into slot 1
    # leaves layer 2's frozen tensor there untouched
    with torch.cuda.stream(sb.inbound):
        buf.fetch_layer_params(2, 1)
        buf.fetch_layer_params(0, 1, skip_frozen=True)
        buf.fetch_layer_grads(1, 0)
        buf.fetch_layer_opt(1, 1)
    sb.synchronize_all()
    assert torch.equal(buf.gpu_param_slot(1, specs[2])["w_frozen_emb"].cpu(), buf.host_params[2]["w_frozen_emb"])
    assert torch.equal(buf.gpu_param_slot(1, specs[0])["w_q"].cpu(), buf.host_params[0]["w_q"])
    assert torch.equal(buf.gpu_grad_slot(0, specs[1])["g_o"].cpu(), buf.host_grads[1]["g_o"])
    assert torch.equal(buf.gpu_opt_slot(1, 1)["o_adam_v_o"].cpu(), buf.host_opt[1]["o_adam_v_o"])
    # offloads write back what the slot holds (params: trainable region only)
    buf.gpu_param_slot(1, specs[0])["w_q"].add_(1.0)
    buf.gpu_param_slot(1, specs[0])["w_frozen_emb"].add_(1.0)
    buf.gpu_grad_slot(0, specs[1])["g_o"].mul_(2.0)
    frozen_before = buf.host_params[0]["w_frozen_emb"].clone()
    want_q = buf.host_params[0]["w_q"] + 1.0
    want_g = buf.host_grads[1]["g_o"] * 2.0
    torch.cuda.synchronize()
    buf.offload_layer_params(0, 1, stream=sb.outbound)
    buf.offload_layer_grads(1, 0, stream=sb.outbound)
    buf.offload_layer_opt(1, 1, stream=sb.outbound, non_blocking=False)
    sb.synchronize_all()
    assert torch.equal(buf.host_params[0]["w_q"], want_q) and torch.equal(buf.host_grads[1]["g_o"], want_g)
    assert torch.equal(buf.host_params[0]["w_frozen_emb"], frozen_before)
    buf.restore_activation_ring()
    buf.release()


@pytest.mark.parametrize("n_layers,n_p,n_g,n_o", [(5, 2, 2, 2), (4, 3, 2, 1), (3, 1, 1, 1), (6, 2, 3, 4), (2, 3, 3, 3)])
@pytest.mark.parametrize("mode", ["flat", "per_tensor", "optimizer_object"])
def test_pipelined_step_equals_synchronous_step_and_oracle(dev, n_layers, n_p, n_g, n_o, mode):
    kw = dict(n_gpu_opt_layers=n_o, step_num=4)
    if mode == "optimizer_object":
        kw["optimizer"] = AdamW(AdamWHyperparams(**HP), state_dtype=torch.float32)
    else:
        kw.update(HP, per_tensor=(mode == "per_tensor"))
    specs, piped = _make(dev, n_layers, n_p, n_g, 7)
    _, sync = _make(dev, n_layers, n_p, n_g, 7)
    before = _snapshot(piped)
    assert ring_optimizer_step(piped, StreamBundle.create(dev), EventBook(), **kw) == 0
    assert ring_optimizer_step(sync, StreamBundle.create(dev), EventBook(), synchronize_every_op=True, **kw) == 0
    for lid in range(n_layers):
        for table in ("host_params", "host_grads", "host_opt"):
            a, b = getattr(piped, table)[lid], getattr(sync, table)[lid]
            for k in a:
                assert torch.equal(a[k], b[k]), f"layer {lid} {table}[{k}]: pipelined != synchronous"
        # oracle: every trainable tensor stepped once; frozen tensors and gradients untouched
        for t in specs[lid].tensors:
            if t.frozen:
                assert torch.equal(piped.host_params[lid][t.name], before[lid]["p"][t.name])
                continue
            gk = "g_" + (t.name[2:] if t.name.startswith("w_") else t.name)
            mk, vk = state_key("o_adam_m", t.name), state_key("o_adam_v", t.name)
            p_ref, m_ref, v_ref, _ = o_adamw.adamw_step(before[lid]["p"][t.name], before[lid]["g"][gk],
                                                        before[lid]["o"][mk], before[lid]["o"][vk], step=4, **HP)
            torch.testing.assert_close(piped.host_params[lid][t.name], p_ref, rtol=1e-4, atol=1e-7)
            torch.testing.assert_close(piped.host_opt[lid][mk], m_ref, rtol=1e-4, atol=1e-7)
            torch.testing.assert_close(piped.host_opt[lid][vk], v_ref, rtol=1e-4, atol=1e-10)
            assert torch.equal(piped.host_grads[lid][gk], before[lid]["g"][gk])
    # a second step straight after the first (rings and events reused)
    assert ring_optimizer_step(piped, StreamBundle.create(dev), EventBook(), **{**kw, "step_num": 5}) == 0
    assert ring_optimizer_step(sync, StreamBundle.create(dev), EventBook(), synchronize_every_op=True,
                               **{**kw, "step_num": 5}) == 0
    for lid in range(n_layers):
        for k in piped.host_params[lid]:
            assert torch.equal(piped.host_params[lid][k], sync.host_params[lid][k])
    piped.release()
    sync.release()


def test_failed_optimizer_status_restores_the_ring(dev):
    specs, buf = _make(dev, 3, 2, 2, 9)
    buf.host_grads[1]["g_q"][3, 3] = float("nan")
    opt = AdamW(AdamWHyperparams(check_error=True, **HP), state_dtype=torch.float32)
    before = buf.host_params[2]["w_q"].clone()
    rc = ring_optimizer_step(buf, StreamBundle.create(dev), EventBook(), n_gpu_opt_layers=2, step_num=1, optimizer=opt)
    assert rc == -1
    with pytest.raises(RuntimeError):
        buf.gpu_opt_slot(0, 0)                                   # back in activation mode
    assert torch.equal(buf.host_params[2]["w_q"], before)        # the step stopped before layer 2
    buf.release()
