"""Activation-slot layout and host logic (CPU): sizes against hand arithmetic for the layout rules
of flextrain/core/activation_schema.py (256-byte field and slot alignment, declaration order,
tier / persist / offload selection), slot views, and the row/pitch description of narrowed views
that the batched copy relies on."""
import pytest
import torch

from flextrain_amd.activation_schema import (
    ActivationField,
    ActivationSchema,
    ActivationSlot,
    _as_rows,
    _match_to,
    concat_fields,
)

bf, f32, i32 = torch.bfloat16, torch.float32, torch.int32
DIMS = {"d": 96, "kv": 32, "H": 3, "F": 200, "E": 5}


def layer_fields():
    return (
        ActivationField("x_inp", lambda T, m: (T, m["d"]), bf, 0),
        ActivationField("attn_norm_rstd", lambda T, m: (T, 1), f32, 0),
        ActivationField("xk", lambda T, m: (T, m["kv"]), bf, 0),
        ActivationField("softmax_lse", lambda T, m: (m["H"], T), f32, 1, token_axis=1),
        ActivationField("xq", lambda T, m: (T, m["d"]), bf, 2),
        ActivationField("router_meta", lambda T, m: (m["E"],), i32, 0, offload=False, token_axis=None),
        ActivationField("scratch", lambda T, m: (T, m["d"]), bf, 0, persist=False),
        ActivationField("x1", lambda T, m: (T, m["F"]), bf, 3),
    )


def up(n, a=256):
    return (n + a - 1) // a * a


def test_sizes_by_hand():
    s = ActivationSchema(layer_fields(), max_tier=3)
    T = 7
    x_inp, rstd, xk, lse, xq, meta, scratch, x1 = T * 96 * 2, T * 4, T * 32 * 2, 3 * T * 4, T * 96 * 2, 5 * 4, T * 96 * 2, T * 200 * 2
    # level 0, persistent: x_inp, rstd, xk, router_meta (each field starts on a 256-byte boundary)
    assert s.home_size_bytes(T, DIMS, 0) == up(up(up(up(x_inp) + rstd) + xk) + meta)
    # level 3: + lse, xq (before router_meta, declaration order), x1 after it; scratch has no home
    off = up(x_inp) + rstd
    off = up(off) + xk
    off = up(off) + lse
    off = up(off) + xq
    off = up(off) + meta
    off = up(off) + x1
    assert s.home_size_bytes(T, DIMS, 3) == up(off)
    # device slot: every field, scratch included
    off = up(x_inp) + rstd
    off = up(off) + xk
    off = up(off) + lse
    off = up(off) + xq
    off = up(off) + meta
    off = up(off) + scratch
    off = up(off) + x1
    assert s.device_size_bytes(T, DIMS) == up(off)
    assert s.offloaded_bytes_at_level(T, DIMS, 0) == x_inp + rstd + xk
    assert s.offloaded_bytes_at_level(T, DIMS, 1) == x_inp + rstd + xk + lse
    assert s.offloaded_bytes_at_level(T, DIMS, 3) == x_inp + rstd + xk + lse + xq + x1
    assert s.home_size_bytes(T, DIMS, -1) == 0 and s.fields_at_level(-1) == ()
    assert [f.name for f in s.offloadable_fields_at_level(2)] == ["x_inp", "attn_norm_rstd", "xk", "softmax_lse", "xq"]
    assert s.has_field("xk") and not s.has_field("nope")


def test_schema_validation():
    with pytest.raises(ValueError):
        ActivationSchema((ActivationField("a", lambda T, m: (T,), bf, 0),) * 2, max_tier=1)
    with pytest.raises(ValueError):
        ActivationSchema((ActivationField("a", lambda T, m: (T,), bf, 2),), max_tier=1)
    with pytest.raises(ValueError):
        concat_fields([layer_fields()[:2], layer_fields()[1:3]])
    assert len(concat_fields([layer_fields()[:2], layer_fields()[2:]])) == 8


def test_from_buffer_views_alignment_and_has():
    s = ActivationSchema(layer_fields(), max_tier=3)
    T = 7
    buf = torch.zeros(s.home_size_bytes(T, DIMS, 2) + 64, dtype=torch.uint8)
    slot, used = ActivationSlot.from_buffer(s, 2, T, DIMS, buf)
    assert used == s.home_size_bytes(T, DIMS, 2)
    assert set(dict(slot.items())) == {"x_inp", "attn_norm_rstd", "xk", "softmax_lse", "xq", "router_meta"}
    assert slot.x_inp.shape == (T, 96) and slot.x_inp.dtype == bf and slot.softmax_lse.shape == (3, T)
    base = buf.data_ptr()
    for _, t in slot.items():
        assert (t.data_ptr() - base) % 256 == 0
    slot.xk.fill_(3.0)       # views alias the buffer and do not overlap
    assert slot.x_inp.float().abs().sum() == 0 and slot.xq.float().abs().sum() == 0
    assert slot.has("xq") and not slot.has("x1") and not slot.has("whatever")
    with pytest.raises(AttributeError):
        slot.x1
    slot.set("extra", torch.ones(2))
    assert slot.has("extra")
    with pytest.raises(ValueError):
        ActivationSlot.from_buffer(s, 3, T, DIMS, buf[:1000])
    with pytest.raises(TypeError):
        ActivationSlot.from_buffer(s, 3, T, DIMS, buf.view(torch.int16))
    # ring slot: non-persistent fields get storage too
    ring = torch.zeros(s.device_size_bytes(T, DIMS), dtype=torch.uint8)
    dev, used = ActivationSlot.from_buffer(s, 3, T, DIMS, ring, include_nonpersistent=True)
    assert used == ring.numel() and dev.has("scratch")


def test_view_for_and_match_to():
    s = ActivationSchema(layer_fields(), max_tier=3)
    Tmax, T = 16, 5
    ring = torch.zeros(s.device_size_bytes(Tmax, DIMS), dtype=torch.uint8)
    dev, _ = ActivationSlot.from_buffer(s, 3, Tmax, DIMS, ring, include_nonpersistent=True)
    v = dev.view_for(T, DIMS)
    assert v.x_inp.shape == (T, 96) and v.softmax_lse.shape == (3, T) and v.router_meta.shape == (5,)
    assert v.x_inp.data_ptr() == dev.x_inp.data_ptr()
    home = torch.zeros(s.home_size_bytes(T, DIMS, 3), dtype=torch.uint8)
    h, _ = ActivationSlot.from_buffer(s, 3, T, DIMS, home)
    assert _match_to(dev.x1, h.x1).shape == (T, 200)
    with pytest.raises(ValueError):
        _match_to(h.x1, dev.x1)


def test_rows_and_pitch_of_narrowed_views():
    t = torch.zeros(6, 10, dtype=bf)
    assert _as_rows(t) == (1, 120, 120)
    assert _as_rows(t[:4]) == (1, 80, 80)                       # a prefix of rows stays contiguous
    assert _as_rows(t[:, :7]) == (6, 14, 20)                    # narrowed inner axis: 6 rows, pitch 20 bytes
    u = torch.zeros(3, 4, 10, dtype=f32)
    assert _as_rows(u[:, :, :5]) == (12, 20, 40)
    assert _as_rows(u[:, :2]) == (3, 80, 160)
    assert _as_rows(u[:, :2, :5]) is None                       # two different pitches: no single 2-D form
    assert _as_rows(torch.zeros(0, 4)) == (0, 0, 0)
    assert _as_rows(t.t()) is None


def test_copy_descriptor_pairs():
    from flextrain_amd.activation_schema import _copy_desc

    full = torch.zeros(6, 10, dtype=bf)
    home = torch.zeros(6, 7, dtype=bf)
    assert _copy_desc(home, full[:, :7]) == (6, 14, 14, 20)          # contiguous home <- narrowed ring view
    assert _copy_desc(full[:, :7], home) == (6, 14, 20, 14)          # and back
    assert _copy_desc(home, home.clone()) == (1, 84, 84, 84)
    other = torch.zeros(6, 12, dtype=bf)
    assert _copy_desc(full[:, :7], other[:, :7]) == (6, 14, 20, 24)  # both pitched, same pieces
    assert _copy_desc(home, full.t()[:7].t()) == (6, 14, 14, 20)
    assert _copy_desc(home.t(), full[:, :7].t()) is None             # transposed views: no 2-D form
