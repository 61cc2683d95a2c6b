"""Pinned host memory, stream/event bookkeeping and the streamed AdamW chunk.
The streamed step must equal the HBM-resident kernel bit for bit (the update is
element-wise, so cutting the chunk into sub-chunks cannot change it) and the CPU oracle
(torch.optim.AdamW semantics) within fp32 rtol 1e-4."""
import types

import pytest
import torch

from flextrain_amd import ops
from flextrain_amd.host_memory import (HostMemoryBackend, LocalPinnedHostBackend, destroy_pinned_tensor, pin_tensor)
from flextrain_amd.optim import (AdamW, AdamWHyperparams, adamw_stream_workspace, flextrain_adamw_step_streamed,
                                 state_key)
from flextrain_amd.streams import EventBook, StreamBundle
from oracle import adamw as o_adamw
from util import gen, randn

pytestmark = pytest.mark.gpu

HP = dict(lr=3e-5, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)


def _state(n, seed, state_dtype=torch.float32):
    g = gen(seed)
    p = randn(g, n, dtype=torch.float32, std=0.02)
    m = randn(g, n, dtype=torch.float32, std=1e-3).to(state_dtype)
    v = (randn(g, n, dtype=torch.float32, std=1e-3) ** 2).to(state_dtype)
    gr = randn(g, n, std=1e-3)
    return p, gr, m, v


def test_pinned_backend_allocates_exact_zeroed_dma_memory(dev):
    be = LocalPinnedHostBackend()
    assert isinstance(be, HostMemoryBackend) and be.name == "local_pinned"
    t = be.allocate_tensor((3, 1000), torch.bfloat16)
    assert t.shape == (3, 1000) and t.dtype == torch.bfloat16 and t.is_pinned() and not t.any()
    t.copy_(torch.arange(3000, dtype=torch.float32).view(3, 1000) / 64)
    d = torch.empty_like(t, device=dev)
    d.copy_(t, non_blocking=True)
    torch.cuda.synchronize()
    assert torch.equal(d.cpu(), t)
    be.release(t)
    be.release(t)          # second release is a no-op
    assert be.allocate_tensor((0,), torch.float32).numel() == 0


def test_pin_tensor_keeps_object_and_values(dev):
    t = torch.arange(1024, dtype=torch.float32)
    same = pin_tensor(t)
    assert same is t and t.is_pinned() and torch.equal(t, torch.arange(1024, dtype=torch.float32))
    d = torch.empty(1024, device=dev)
    d.copy_(t, non_blocking=True)
    torch.cuda.synchronize()
    assert torch.equal(d.cpu(), t)
    destroy_pinned_tensor(t)


def test_stream_bundle_and_event_book(dev):
    sb = StreamBundle.create(dev, with_secondary=True)
    ptrs = {s.cuda_stream for s in (sb.compute, sb.inbound, sb.outbound, sb.inbound_fwd_context, sb.secondary_compute)}
    assert len(ptrs) == 5 and 0 not in ptrs
    book = EventBook()
    x = torch.zeros(1 << 20, device=dev)
    with torch.cuda.stream(sb.inbound):
        x.add_(1.0)
        book.weight_inbound.record_on(7, sb.inbound)
    book.weight_inbound.wait_on(7, sb.compute)
    with torch.cuda.stream(sb.compute):
        y = x * 2
    sb.synchronize_all()
    assert float(y.min()) == 2.0
    book.weight_inbound.mark_consumed(7)
    book.weight_inbound.wait_on(7, sb.compute)           # consumed: no wait, no error
    with pytest.raises(KeyError):
        book.opt_inbound.wait_on(1, sb.compute)
    book.grad_weight_inbound.record_on(1, sb.compute)
    book.dev_act_slot_mapping[(0, 0)] = 3
    book.clear_per_round()
    assert len(book.grad_weight_inbound) == 0 and not book.dev_act_slot_mapping and 7 in book.weight_inbound
    assert StreamBundle.create(dev).secondary_compute is None


@pytest.mark.parametrize("n,sub,slots", [(1_000_003, 65536, 3), (200_000, 1 << 20, 2), (8 * 70_001, 8 * 1000, 4),
                                         (5, 64, 1)])
@pytest.mark.parametrize("state_dtype,copy_to", [(torch.float32, "host"), (torch.bfloat16, "device"),
                                                 (torch.float32, None)])
def test_streamed_step_equals_resident_kernel_and_oracle(dev, n, sub, slots, state_dtype, copy_to):
    p, gr, m, v = _state(n, n % 97, state_dtype)
    be = LocalPinnedHostBackend()
    host = {}
    for name, t in (("p", p), ("g", gr), ("m", m), ("v", v)):
        host[name] = be.allocate_tensor((n,), t.dtype)
        host[name].copy_(t)
    pc = None
    if copy_to == "host":
        pc = be.allocate_tensor((n,), torch.bfloat16)
    elif copy_to == "device":
        pc = torch.zeros(n, dtype=torch.bfloat16, device=dev)
    sb = StreamBundle.create(dev)
    rc = flextrain_adamw_step_streamed(host["p"], host["g"], host["m"], host["v"], streams=sb, step=4,
                                       params_bf16_out=pc, sub_elems=sub, n_slots=slots, **HP)
    assert rc == 0
    sb.synchronize_all()
    # resident kernel on the same inputs
    pd, gd, md, vd = p.to(dev), gr.to(dev), m.to(dev), v.to(dev)
    pcd = torch.empty(n, dtype=torch.bfloat16, device=dev)
    ops.flextrain_adamw_step(pd, gd, md, vd, step=4, params_bf16_out=pcd, **HP)
    assert torch.equal(host["p"], pd.cpu()) and torch.equal(host["m"], md.cpu()) and torch.equal(host["v"], vd.cpu())
    assert torch.equal(host["g"], gr)                                   # gradients are read-only
    if pc is not None:
        assert torch.equal(pc.cpu(), pcd.cpu())
    # oracle
    p_ref, m_ref, v_ref, _ = o_adamw.adamw_step(p, gr, m, v, step=4, **HP)
    torch.testing.assert_close(host["p"], p_ref, rtol=1e-4, atol=1e-7)
    if state_dtype == torch.float32:
        torch.testing.assert_close(host["m"], m_ref, rtol=1e-4, atol=1e-7)
        torch.testing.assert_close(host["v"], v_ref, rtol=1e-4, atol=1e-10)
    for t in host.values():
        be.release(t)


def _pinned_state(be, n, seed, step_fill=None):
    p, gr, m, v = _state(n, seed)
    host = {}
    for name, t in (("p", p), ("g", gr), ("m", m), ("v", v)):
        host[name] = be.allocate_tensor((n,), t.dtype)
        host[name].copy_(t)
    host["pc"] = be.allocate_tensor((n,), torch.bfloat16)
    return (p, gr, m, v), host


def _resident(dev, state, step):
    p, gr, m, v = (t.to(dev) for t in state)
    pc = torch.empty(p.numel(), dtype=torch.bfloat16, device=dev)
    ops.flextrain_adamw_step(p, gr, m, v, step=step, params_bf16_out=pc, **HP)
    return p.cpu(), m.cpu(), v.cpu(), pc.cpu()


@pytest.mark.parametrize("raw_workspace", [False, True])
def test_back_to_back_calls_on_one_workspace_need_no_sync(dev, raw_workspace):
    """Successive chunks (the engine's layer-after-layer pattern) through ONE staging workspace with
    nothing between the calls: the second call's copies-in must not overwrite slots the first call's
    kernels and copies-out still use.  Three chunks of different sizes, each several rounds of the
    slots, then one more step on the first chunk; every host buffer equals the resident kernel."""
    be = LocalPinnedHostBackend()
    sb = StreamBundle.create(dev)
    sub, slots = 64 * 1024, 3
    sizes = (1_500_003 // 8 * 8, 700_000, 1_000_003)
    chunks = [_pinned_state(be, n, 300 + i) for i, n in enumerate(sizes)]
    ws = adamw_stream_workspace(sub, slots, torch.float32, torch.bfloat16, torch.float32, True, dev)
    if raw_workspace:
        ws = ws.buffer                          # no ring: every call fences on compute / outbound instead
    for state, host in chunks:
        flextrain_adamw_step_streamed(host["p"], host["g"], host["m"], host["v"], streams=sb, step=4,
                                      params_bf16_out=host["pc"], workspace=ws, sub_elems=sub, n_slots=slots, **HP)
    state0, host0 = chunks[0]
    flextrain_adamw_step_streamed(host0["p"], host0["g"], host0["m"], host0["v"], streams=sb, step=5,
                                  params_bf16_out=host0["pc"], workspace=ws, sub_elems=sub, n_slots=slots, **HP)
    sb.synchronize_all()
    for i, (state, host) in enumerate(chunks):
        p, m, v, pc = _resident(dev, state, 4)
        if i == 0:
            p, m, v, pc = _resident(dev, (p, state[1], m, v), 5)
        assert torch.equal(host["p"], p) and torch.equal(host["m"], m) and torch.equal(host["v"], v), f"chunk {i}"
        assert torch.equal(host["pc"], pc), f"chunk {i} bf16 copy"
    for _, host in chunks:
        for t in host.values():
            be.release(t)


def test_streamed_step_full_llama_layer_chunk(dev):
    """218,112,000 parameters (one Llama-3.1-8B decoder layer): fp32 p/m/v + bf16 g in pinned host
    memory, 3 slots x 4 Mi elements, bf16 copy-out to pinned host.  Bit-equal to the resident kernel
    on all elements; against the oracle on a strided sample (rtol 1e-4)."""
    n = 218_112_000
    be = LocalPinnedHostBackend()
    g = gen(1003)
    host = dict(p=be.allocate_tensor((n,), torch.float32), g=be.allocate_tensor((n,), torch.bfloat16),
                m=be.allocate_tensor((n,), torch.float32), v=be.allocate_tensor((n,), torch.float32),
                pc=be.allocate_tensor((n,), torch.bfloat16))
    host["p"].normal_(0, 0.02, generator=g)
    host["g"].copy_(torch.empty(n).normal_(0, 1e-3, generator=g))
    host["m"].normal_(0, 1e-3, generator=g)
    host["v"].normal_(0, 1e-3, generator=g).square_()
    sample = torch.arange(0, n, 997)
    before = {k: host[k][sample].clone() for k in ("p", "g", "m", "v")}
    pd, gd, md, vd = (host[k].to(dev) for k in ("p", "g", "m", "v"))
    pcd = torch.empty(n, dtype=torch.bfloat16, device=dev)
    ops.flextrain_adamw_step(pd, gd, md, vd, step=4, params_bf16_out=pcd, **HP)
    sb = StreamBundle.create(dev)
    assert flextrain_adamw_step_streamed(host["p"], host["g"], host["m"], host["v"], streams=sb, step=4,
                                         params_bf16_out=host["pc"], **HP) == 0
    sb.synchronize_all()
    for k, d in (("p", pd), ("m", md), ("v", vd), ("pc", pcd)):
        assert torch.equal(host[k].to(dev), d), k
    p_ref, m_ref, v_ref, _ = o_adamw.adamw_step(before["p"], before["g"], before["m"], before["v"], step=4, **HP)
    torch.testing.assert_close(host["p"][sample], p_ref, rtol=1e-4, atol=1e-7)
    torch.testing.assert_close(host["m"][sample], m_ref, rtol=1e-4, atol=1e-7)
    torch.testing.assert_close(host["v"][sample], v_ref, rtol=1e-4, atol=1e-10)
    for t in host.values():
        be.release(t)


def test_streamed_step_rejects_unpinned_and_mismatched(dev):
    sb = StreamBundle.create(dev)
    be = LocalPinnedHostBackend()
    p = be.allocate_tensor((64,), torch.float32)
    g = be.allocate_tensor((64,), torch.bfloat16)
    m = be.allocate_tensor((64,), torch.float32)
    v = be.allocate_tensor((64,), torch.float32)
    with pytest.raises(ValueError):
        flextrain_adamw_step_streamed(torch.zeros(64), g, m, v, streams=sb)
    with pytest.raises(ValueError):
        flextrain_adamw_step_streamed(p, g, m[:32], v, streams=sb)
    with pytest.raises(TypeError):
        flextrain_adamw_step_streamed(p, g, m, be.allocate_tensor((64,), torch.bfloat16), streams=sb)
    assert flextrain_adamw_step_streamed(p[:0], g[:0], m[:0], v[:0], streams=sb) == 0


def test_adamw_optimizer_object_loops_over_param_spec(dev):
    spec = types.SimpleNamespace(tensors=[types.SimpleNamespace(name="w_q", frozen=False),
                                          types.SimpleNamespace(name="w_frozen", frozen=True),
                                          types.SimpleNamespace(name="final_norm", frozen=False)])
    assert state_key("o_adam_m", "w_q") == "o_adam_m_q" and state_key("o_adam_v", "final_norm") == "o_adam_v_final_norm"
    master, grads, state, want = {}, {}, {}, {}
    for i, (w, gk) in enumerate((("w_q", "g_q"), ("w_frozen", "g_frozen"), ("final_norm", "g_final_norm"))):
        p, gr, m, v = _state(4096, 50 + i)
        master[w], grads[gk] = p.to(dev), gr.to(dev)
        state[state_key("o_adam_m", w)], state[state_key("o_adam_v", w)] = m.to(dev), v.to(dev)
        want[w] = o_adamw.adamw_step(p, gr, m, v, step=2, **HP)[0] if w != "w_frozen" else p
    opt = AdamW(AdamWHyperparams(**HP), state_dtype=torch.float32)
    assert opt.step(spec, master, grads, state, step_num=2) == 0
    for w in master:
        torch.testing.assert_close(master[w].cpu(), want[w], rtol=1e-4, atol=1e-7)
    grads["g_q"][5] = float("nan")
    bad = AdamW(AdamWHyperparams(check_error=True, **HP))
    assert bad.step(spec, master, grads, state, step_num=3) == -1
