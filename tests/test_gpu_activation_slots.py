"""send_home / fetch_home of tiered activation slots between the HBM ring (sized for the largest
chunk) and pinned home slots (sized for the chunk): byte-exact round trips per save level, fields
outside the level or not offloadable left alone, and the engine's stream / event protocol."""
import pytest
import torch

from flextrain_amd.activation_schema import (
    ActivationField,
    ActivationSchema,
    ActivationSlot,
    ActivationStreamer,
    fetch_home,
    send_home,
)
from flextrain_amd.host_memory import LocalPinnedHostBackend
from flextrain_amd.streams import EventBook, StreamBundle

pytestmark = pytest.mark.gpu

bf, f32, i32 = torch.bfloat16, torch.float32, torch.int32
DIMS = {"d": 512, "kv": 128, "H": 4, "F": 1408, "E": 8, "K": 2}


def schema():
    return ActivationSchema((
        ActivationField("x_inp", lambda T, m: (T, m["d"]), bf, 0),
        ActivationField("attn_norm_rstd", lambda T, m: (T, 1), f32, 0),
        ActivationField("xk", lambda T, m: (T, m["kv"]), bf, 0),
        ActivationField("softmax_lse", lambda T, m: (m["H"], T), f32, 1, token_axis=1),
        ActivationField("xq", lambda T, m: (T, m["d"]), bf, 2),
        ActivationField("router_meta", lambda T, m: (m["E"],), i32, 0, offload=False, token_axis=None),
        ActivationField("x_up", lambda T, m: (T * m["K"], 2 * m["F"]), bf, 3, token_axis=None),
        ActivationField("scratch", lambda T, m: (T, m["d"]), bf, 0, persist=False),
        ActivationField("x1", lambda T, m: (T, m["F"]), bf, 3),
    ), max_tier=3)


def _fill(slot, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    for name, t in slot.items():
        src = torch.randint(-1000, 1000, tuple(t.shape), generator=g).to(t.dtype)
        t.copy_(src)


@pytest.mark.parametrize("level", [0, 1, 2, 3])
@pytest.mark.parametrize("T,Tmax", [(300, 512), (512, 512), (1, 64)])
def test_round_trip_per_level(dev, level, T, Tmax):
    s = schema()
    pinned = LocalPinnedHostBackend()
    ring = torch.zeros(s.device_size_bytes(Tmax, DIMS), dtype=torch.uint8, device=dev)
    full, used = ActivationSlot.from_buffer(s, s.max_tier, Tmax, DIMS, ring, include_nonpersistent=True)
    assert used == ring.numel()
    _fill(full, 7)
    computed = full.view_for(T, DIMS)
    home_buf = pinned.allocate_tensor((s.home_size_bytes(T, DIMS, level),), torch.uint8)
    home_buf.fill_(0xAB)
    home, _ = ActivationSlot.from_buffer(s, level, T, DIMS, home_buf)
    send_home(home, computed, level, non_blocking=False)
    names = [f.name for f in s.offloadable_fields_at_level(level)]
    for n in names:
        want = getattr(full, n)
        hv = getattr(home, n)
        for ax, (a, b) in enumerate(zip(want.shape, hv.shape)):
            want = want.narrow(ax, 0, b)
        assert torch.equal(hv, want.cpu()), n
    if level >= 0:     # not offloadable: the home view keeps its fill pattern
        assert torch.equal(home.router_meta.view(torch.uint8), torch.full((32,), 0xAB, dtype=torch.uint8))

    # wipe the ring, fetch back, compare the offloaded fields; everything else stays wiped
    snapshot = {n: getattr(full, n).clone() for n in names}
    ring.zero_()
    dest = ActivationSlot(s, level, {n: full._tensors[n] for n in names})
    fetch_home(dest, home, level, non_blocking=False)
    for n in names:
        got, want = getattr(full, n), snapshot[n]
        hv = getattr(home, n)
        sub_g, sub_w = got, want
        for ax, b in enumerate(hv.shape):
            sub_g, sub_w = sub_g.narrow(ax, 0, b), sub_w.narrow(ax, 0, b)
        assert torch.equal(sub_g, sub_w), n
    others = [n for n, _ in full.items() if n not in names]
    for n in others:
        assert not getattr(full, n).any(), n
    total = sum(int(getattr(full, n).ne(0).sum()) for n in names)
    assert total > 0 or T == 0
    pinned.release(home_buf)


def test_schema_mismatch_and_too_small_source(dev):
    s1, s2 = schema(), schema()
    b = torch.zeros(s1.device_size_bytes(8, DIMS), dtype=torch.uint8, device=dev)
    a, _ = ActivationSlot.from_buffer(s1, 3, 8, DIMS, b, include_nonpersistent=True)
    h = torch.zeros(s2.home_size_bytes(8, DIMS, 3), dtype=torch.uint8).pin_memory()
    c, _ = ActivationSlot.from_buffer(s2, 3, 8, DIMS, h)
    with pytest.raises(ValueError):
        send_home(c, a, 3)
    with pytest.raises(ValueError):
        fetch_home(a, c, 3)
    h16 = torch.zeros(s1.home_size_bytes(16, DIMS, 3), dtype=torch.uint8).pin_memory()
    big, _ = ActivationSlot.from_buffer(s1, 3, 16, DIMS, h16)
    with pytest.raises(ValueError):
        send_home(big, a, 3)          # the device slot holds fewer tokens than the home slot wants


def test_streamer_offload_then_prefetch_into_another_ring_slot(dev):
    s = schema()
    T, Tmax, level = 200, 256, 1
    streams, events = StreamBundle.create(dev), EventBook()
    st = ActivationStreamer(streams, events)
    slot_bytes = s.device_size_bytes(Tmax, DIMS)
    ring = torch.zeros(2 * slot_bytes, dtype=torch.uint8, device=dev)
    slot0, _ = ActivationSlot.from_buffer(s, 3, Tmax, DIMS, ring[:slot_bytes], include_nonpersistent=True)
    slot1, _ = ActivationSlot.from_buffer(s, 3, Tmax, DIMS, ring[slot_bytes:], include_nonpersistent=True)
    pinned = LocalPinnedHostBackend()
    home_buf = pinned.allocate_tensor((s.home_size_bytes(T, DIMS, level),), torch.uint8)
    home, _ = ActivationSlot.from_buffer(s, level, T, DIMS, home_buf)
    key = (3, 0)
    with torch.cuda.stream(streams.compute):
        computed = slot0.view_for(T, DIMS)
        computed.x_inp.fill_(1.5)                     # "forward" produces the fields on the compute stream
        computed.softmax_lse.fill_(-2.0)
        computed.xq.fill_(9.0)                        # tier 2: not saved at level 1
    st.offload(key, 0, home, computed, level)
    assert key in events.home_act_slot_available and 0 in events.act_slot_ready
    with torch.cuda.stream(streams.compute):
        events.act_slot_ready.wait_on(0, streams.compute)
        ring[:slot_bytes].zero_()                      # the ring slot is reused
    dev_slot = st.prefetch(key, slot1.view_for(T, DIMS), home)
    events.inbound_act_slot_ready.wait_on(key, streams.compute)
    streams.synchronize_all()
    assert events.dev_act_slot_mapping[key] is dev_slot and dev_slot.level == level
    assert dev_slot.has("x_inp") and dev_slot.has("softmax_lse") and not dev_slot.has("xq")
    assert torch.all(dev_slot.x_inp == 1.5) and torch.all(dev_slot.softmax_lse == -2.0)
    assert not dev_slot.xq.any()                       # stale / unfetched: still the ring's zeros
    assert torch.all(home.x_inp == 1.5)
    pinned.release(home_buf)
