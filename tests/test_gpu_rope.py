"""HIP rotary embedding against the CPU oracle (bf16 rtol = atol = 1e-2)."""
import pytest
import torch

from flextrain_amd import ops
from oracle import rope as o_rope
from util import close, gen, randn

pytestmark = pytest.mark.gpu


def _positions(kind, T, g):
    if kind == "arange":
        return torch.arange(T, dtype=torch.int32).view(T, 1)
    if kind == "packed":  # small sequences restart at 0 inside a chunk (engine/schedule.py:358-374)
        return (torch.arange(T, dtype=torch.int32) % 37).view(T, 1)
    if kind == "continuation":  # later chunk of a long sequence (engine/schedule.py:377-401)
        return (torch.arange(T, dtype=torch.int32) + 123456).view(T, 1)
    return torch.randint(0, 131072, (T, 1), generator=g, dtype=torch.int32)


@pytest.mark.parametrize("kind", ["arange", "packed", "continuation", "random"])
@pytest.mark.parametrize("T,Hq,Hk,D", [(512, 32, 8, 128), (100, 4, 4, 64), (33, 3, 1, 256), (7, 1, 1, 16),
                                       (37, 6, 6, 128),      # 3 chunks of 64 packs per token: a wave's two chunks straddle tokens
                                       (101, 4, 4, 64),      # one chunk per token, odd chunk count
                                       (19, 5, 2, 128)])     # 7 heads: not a whole number of 64-pack chunks (workgroup kernel)
def test_fwd_bwd_fused(dev, kind, T, Hq, Hk, D):
    g = gen(1010)
    q, k = randn(g, T, Hq, D), randn(g, T, Hk, D)
    pos = _positions(kind, T, g)
    inv = o_rope.vanilla_inv_freq(D, 500000.0)
    theta = torch.tensor([500000.0])
    for backward in (False, True):
        qd, kd = q.to(dev), k.to(dev)
        fn = ops.flextrain_rope_bwd if backward else ops.flextrain_rope_fwd
        out = fn([qd, kd], pos.to(dev), theta)
        assert out[0] is qd and out[1] is kd
        close(qd, o_rope.rope(q, pos, inv, backward), what=f"q bwd={backward}")
        close(kd, o_rope.rope(k, pos, inv, backward), what=f"k bwd={backward}")


def test_full_size_q_k_and_roundtrip(dev):
    """The Llama-3.1-8B shape: q [8192,32,128], k [8192,8,128], theta 5e5."""
    g = gen(1001)
    T = 8192
    q, k = randn(g, T, 32, 128), randn(g, T, 8, 128)
    pos = torch.arange(T, dtype=torch.int32).view(T, 1)
    inv = o_rope.vanilla_inv_freq(128, 500000.0)
    qd, kd, pd, fd = q.to(dev), k.to(dev), pos.to(dev), inv.to(dev)
    ops.flextrain_rope_fwd([qd, kd], pd, fd)
    close(qd, o_rope.rope(q, pos, inv), what="q")
    close(kd, o_rope.rope(k, pos, inv), what="k")
    # isometry per pair (size-independent property), then inverse rotation
    n_in = q.float().reshape(T, 32, 64, 2).norm(dim=-1)
    n_out = qd.float().cpu().reshape(T, 32, 64, 2).norm(dim=-1)
    torch.testing.assert_close(n_out, n_in, rtol=2e-2, atol=2e-2)
    ops.flextrain_rope_bwd([qd, kd], pd, fd)
    close(qd, q, rtol=2e-2, atol=2e-2, what="bwd(fwd(q))")
    close(kd, k, rtol=2e-2, atol=2e-2, what="bwd(fwd(k))")


def test_fused_equals_separate_and_lists(dev):
    g = gen(4)
    T = 64
    ts = [randn(g, T, h, 64) for h in (4, 2, 3)]
    pos = _positions("random", T, g)
    inv = ops.build_rope_inv_freq(64, 10000.0, {"rope_type": "llama3", "factor": 8.0})
    fused = [t.to(dev) for t in ts]
    ops.flextrain_rope_fwd(fused, pos.to(dev), inv.to(dev))
    for t, f in zip(ts, fused):
        single = t.to(dev)
        ops.flextrain_rope_fwd([single], pos.to(dev), inv.to(dev))
        assert torch.equal(single, f)
        close(f, o_rope.rope(t, pos, inv))
    assert ops.flextrain_rope_fwd([], pos.to(dev), inv.to(dev)) == []


def test_strided_views_and_other_dtypes(dev):
    g = gen(5)
    T, H, D = 40, 6, 64
    pos = _positions("random", T, g)
    inv = o_rope.vanilla_inv_freq(D, 10000.0)
    # q sliced out of a fused qkv buffer: token stride 3*H*D (vector path) ...
    qkv = randn(g, T, 3 * H * D)
    qkv_d = qkv.to(dev)
    view = qkv_d.view(T, 3 * H, D)[:, :H, :]
    ops.flextrain_rope_fwd([view], pos.to(dev), inv.to(dev))
    close(view, o_rope.rope(qkv.view(T, 3 * H, D)[:, :H, :], pos, inv))
    assert torch.equal(qkv_d.view(T, 3 * H, D)[:, H:, :].cpu(), qkv.view(T, 3 * H, D)[:, H:, :])
    # ... and a transposed layout with non-unit channel stride (generic path)
    x = randn(g, T, D, H)
    xd = x.to(dev)
    ops.flextrain_rope_fwd([xd.permute(0, 2, 1)], pos.to(dev), inv.to(dev))
    close(xd.permute(0, 2, 1), o_rope.rope(x.permute(0, 2, 1), pos, inv))
    for dtype, tol in ((torch.float32, 2e-3), (torch.float16, 1e-2)):
        y = randn(g, T, H, D, dtype=dtype)
        yd = y.to(dev)
        ops.flextrain_rope_fwd([yd], pos.to(dev), inv.to(dev))
        close(yd, o_rope.rope(y, pos, inv), rtol=tol, atol=tol, what=str(dtype))


def test_partial_rotation(dev):
    g = gen(6)
    T, H, D, rd = 50, 4, 256, 64
    q = randn(g, T, H, D)
    pos = _positions("continuation", T, g)
    inv = o_rope.vanilla_inv_freq(rd, 10000000.0)
    qd = q.to(dev)
    ops.flextrain_rope_partial_fwd([qd], pos.to(dev), torch.tensor([10000000.0]), rd)
    close(qd, o_rope.rope(q, pos, inv, rot_dim=rd))
    assert torch.equal(qd[..., rd:].cpu(), q[..., rd:])
    ops.flextrain_rope_partial_bwd([qd], pos.to(dev), inv.to(dev), rd)
    close(qd, q, rtol=2e-2, atol=2e-2)


def test_bad_freqs_length(dev):
    q = torch.zeros(4, 2, 64, device=dev, dtype=torch.bfloat16)
    pos = torch.zeros(4, 1, device=dev, dtype=torch.int32)
    with pytest.raises(ValueError):
        ops.flextrain_rope_fwd([q], pos, torch.ones(7, device=dev))
