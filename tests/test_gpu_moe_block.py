"""Grouped expert GEMMs and the whole routed-SwiGLU block (reference interface:
flextrain/ops/full_moe.py, flextrain/ops/moe_backend.py) against the CPU oracle.
Tolerances: bf16 tensors rtol = atol = 1e-2 scaled to the tensor's magnitude where
GEMM sums grow it, plus the reference's own gate cos >= 0.999
(tests/moe/test_moe_backend_parity.py:251-389)."""
import types

import pytest
import torch

from flextrain_amd import full_moe
from flextrain_amd.moe_backend import FlextrainMoEExpertCompute, MoEExpertCompute
from flextrain_amd.ops.grouped import flextrain_grouped_gemm_rows, flextrain_grouped_gemm_wgrad
from oracle import moe as o_moe
from util import gen, randn

pytestmark = pytest.mark.gpu


def _cos(a, b):
    a, b = a.float().flatten().cpu(), b.float().flatten().cpu()
    return float(torch.nn.functional.cosine_similarity(a, b, dim=0))


def _close_scaled(got, want, what, tol=1e-2):
    """|got - want| <= tol*|want| + tol*max(1, rms(want)): the stated bf16 tolerance with
    the absolute part scaled to the tensor's magnitude (GEMM sums are not O(1)), plus
    the reference's cosine gate."""
    got, want = got.float().cpu(), want.float().cpu()
    floor = tol * max(1.0, float(want.pow(2).mean().sqrt()))
    bad = (got - want).abs() > tol * want.abs() + floor
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.numel()} outside tolerance, max abs err " \
                          f"{float((got - want).abs().max()):.4g}, floor {floor:.4g}"
    if want.numel() > 1 and float(want.abs().max()) > 0:
        assert _cos(got, want) >= 0.999, f"{what}: cos {_cos(got, want)}"


def _ragged_counts(g, E, TK):
    w = torch.rand(E, generator=g)
    w[1] = 0.0                                  # an expert without rows
    c = torch.floor(w / w.sum() * TK).to(torch.int32)
    c[0] += TK - int(c.sum())
    return c


@pytest.mark.parametrize("E,TK,K,N", [(8, 1000, 256, 384), (128, 65536, 2048, 1536), (4, 300, 64, 72), (3, 50, 8, 8),
                                      (5, 700, 96, 520),       # K a multiple of 32 only, N not a multiple of the tile
                                      (3, 200, 32, 40),        # a single 32-wide K-step
                                      (3, 5000, 160, 264)])    # large experts: 256-row tiles, K tail of 32
@pytest.mark.parametrize("trans_b", [True, False])
def test_grouped_rows(dev, E, TK, K, N, trans_b):
    g = gen(E * 13 + N)
    counts = _ragged_counts(g, E, TK)
    A = randn(g, TK, K, std=0.5)
    W = randn(g, E, N, K, std=0.1) if trans_b else randn(g, E, K, N, std=0.1)
    Bd = W.to(dev).transpose(1, 2) if trans_b else W.to(dev)
    D = torch.full((TK, N), 7.0, dtype=torch.bfloat16, device=dev)
    flextrain_grouped_gemm_rows(A.to(dev), Bd, counts.to(dev), D)
    off = o_moe.expert_offsets(counts)
    experts = range(E) if E <= 8 else (0, 1, 2, 17, 63, 127)
    for e in experts:
        a, b = int(off[e]), int(off[e + 1])
        if a == b:
            continue
        Be = W[e].float().t() if trans_b else W[e].float()
        _close_scaled(D[a:b], A[a:b].float() @ Be, f"expert {e}")
    assert int(off[-1]) == TK
    # beta/C path, counts in pinned host memory
    C = randn(g, TK, N)
    D2 = C.to(dev).clone()
    flextrain_grouped_gemm_rows(A.to(dev), Bd, counts.pin_memory(), D2, C=D2, alpha=0.5, beta=1.0)
    e = 0
    a, b = int(off[e]), int(off[e + 1])
    Be = W[e].float().t() if trans_b else W[e].float()
    _close_scaled(D2[a:b], 0.5 * (A[a:b].float() @ Be) + C[a:b].float(), "beta path")


def test_grouped_rows_fp16(dev):
    g = gen(77)
    E, TK, K, N = 6, 900, 128, 200
    counts = _ragged_counts(g, E, TK)
    A = randn(g, TK, K, std=0.5, dtype=torch.float16)
    W = randn(g, E, N, K, std=0.1, dtype=torch.float16)
    D = torch.empty((TK, N), dtype=torch.float16, device=dev)
    flextrain_grouped_gemm_rows(A.to(dev), W.to(dev).transpose(1, 2), counts.to(dev), D)
    off = o_moe.expert_offsets(counts)
    for e in range(E):
        a, b = int(off[e]), int(off[e + 1])
        if a < b:
            _close_scaled(D[a:b], A[a:b].float() @ W[e].float().t(), f"expert {e}")


@pytest.mark.parametrize("E,TK,M,N", [(8, 1000, 256, 384), (128, 65536, 1536, 2048), (4, 300, 64, 72)])
@pytest.mark.parametrize("gdt", [torch.bfloat16, torch.float32])
def test_grouped_wgrad_accumulates(dev, E, TK, M, N, gdt):
    g = gen(E + M)
    counts = _ragged_counts(g, E, TK)
    A, B = randn(g, TK, M, std=0.5), randn(g, TK, N, std=0.5)
    G0 = randn(g, E, M, N, dtype=gdt)
    G = G0.to(dev).clone()
    flextrain_grouped_gemm_wgrad(A.to(dev), B.to(dev), G, counts.to(dev))          # beta = 1: accumulate
    off = o_moe.expert_offsets(counts)
    experts = range(E) if E <= 8 else (0, 1, 5, 127)
    for e in experts:
        a, b = int(off[e]), int(off[e + 1])
        want = G0[e].float() + A[a:b].float().t() @ B[a:b].float()
        _close_scaled(G[e], want, f"expert {e}")
    assert torch.equal(G[1].cpu(), G0[1]), "expert without rows must keep its accumulator"
    G2 = torch.full_like(G, 3.0)
    flextrain_grouped_gemm_wgrad(A.to(dev), B.to(dev), G2, counts.to(dev), beta=0.0)
    assert not G2[1].any(), "beta = 0 overwrites, also for an expert without rows"


def _slot(T, K, E, F, dtype, dev):
    TK = T * K
    return types.SimpleNamespace(
        x_router=torch.empty(T, E, dtype=dtype, device=dev),
        chosen_experts=torch.empty(T, K, dtype=torch.int32, device=dev),
        router_weights=torch.empty(T, K, dtype=dtype, device=dev),
        index_mapping=torch.empty(T, K, dtype=torch.int32, device=dev),
        expert_counts=torch.empty(E, dtype=torch.int32, device=dev),
        scattered_router_weights=torch.empty(TK, 1, dtype=dtype, device=dev),
        x_up=torch.empty(TK, 2 * F, dtype=dtype, device=dev),
        aux={},
    )


def _run_block(dev, T, d, E, K, F, seed, lb=0.0, experts=None, init_grads=False):
    g = gen(seed)
    bf = torch.bfloat16
    x, dy, res = randn(g, T, d), randn(g, T, d), randn(g, T, d)
    w_router = randn(g, d, E, std=0.02)                 # reference layout (d_model, E)
    w_up, w_down = randn(g, E, 2 * F, d, std=0.02), randn(g, E, d, F, std=0.02)
    weights = {k: v.to(dev) for k, v in dict(w_router=w_router, w_up=w_up, w_down=w_down).items()}
    g0 = dict(g_up=randn(g, E, 2 * F, d, std=0.01), g_down=randn(g, E, d, F, std=0.01),
              g_router=randn(g, d, E, std=0.01)) if init_grads else None
    grads = {k: (g0[k].to(dev).clone() if g0 else torch.zeros_like(weights["w" + k[1:]])) for k in
             ("g_up", "g_down", "g_router")}
    slot = _slot(T, K, E, F, bf, dev)
    backend = FlextrainMoEExpertCompute()
    assert isinstance(backend, MoEExpertCompute)
    stream = torch.cuda.current_stream()
    scratch = lambda shape, dtype: torch.empty(shape, dtype=dtype, device=dev)
    out = torch.empty(T, d, dtype=bf, device=dev)
    chunk_extra = {}
    common = dict(slot=slot, chunk_extra=chunk_extra, layer_id=3, primary_stream=stream, secondary_stream=None,
                  scratch_fn=scratch, expert_compute=backend)
    full_moe.routed_swiglu_moe_fwd(x.to(dev), weights, out_tensor=out, residual=res.to(dev), top_k=K, num_experts=E,
                                   routing_mode="topk_then_softmax", **common)
    dx = full_moe.routed_swiglu_moe_bwd(dy.to(dev), weights, grads, slot, chunk_extra, 3, ffn_norm_output=x.to(dev),
                                        top_k=K, num_experts=E, routing_mode="topk_then_softmax",
                                        load_balance_coef=lb, total_tokens_per_step=4 * T if lb else None,
                                        primary_stream=stream, secondary_stream=None, scratch_fn=scratch,
                                        expert_compute=backend)
    torch.cuda.synchronize()
    logits = slot.x_router.cpu()                         # routing is exact only from identical logits
    ref = o_moe.routed_block_fwd_bwd(x, logits, w_router, w_up, w_down, res, dy, K, load_balance_coef=lb,
                                     tokens_per_step=4 * T if lb else None, experts=experts)
    return dict(out=out, dx=dx, grads=grads, slot=slot, ref=ref, g0=g0, x=x, w_router=w_router, res=res, dy=dy,
                weights_cpu=dict(w_router=w_router, w_up=w_up, w_down=w_down),
                host_counts=chunk_extra[backend._CHUNK_EXTRA_HOST_COUNTS][3])


@pytest.mark.parametrize("T,d,E,K,F,lb,init", [(128, 128, 8, 2, 64, 0.0, False), (1024, 512, 32, 8, 256, 0.01, True),
                                               (300, 256, 16, 4, 96, 0.0, True)])
def test_block_fwd_bwd(dev, T, d, E, K, F, lb, init):
    r = _run_block(dev, T, d, E, K, F, seed=1009, lb=lb, init_grads=init)
    ref, slot = r["ref"], r["slot"]
    # router GEMM under float tolerance; everything downstream from identical logits
    want_logits = r["x"].float() @ r["w_router"].float()
    _close_scaled(slot.x_router, want_logits, "router logits")
    assert torch.equal(slot.chosen_experts.cpu(), ref["ids"])
    assert torch.equal(slot.index_mapping.cpu(), ref["mapping"])
    assert torch.equal(slot.expert_counts.cpu(), ref["counts"])
    assert torch.equal(r["host_counts"], ref["counts"])
    _close_scaled(r["out"], ref["out"], "out")
    _close_scaled(slot.x_up, ref["pre"], "x_up (saved pre-activation)")
    _close_scaled(r["dx"], ref["dx"], "dx")
    for name in ("g_up", "g_down", "g_router"):
        want = ref[name] + (r["g0"][name].float() if r["g0"] else 0.0)
        _close_scaled(r["grads"][name], want, name)
    assert "moe_dprobs" not in slot.aux


def _check_sampled_block(dev, T, d, E, K, F, picks, seed, n_tokens=64):
    """The oracle evaluates the experts in ``picks`` (their row ranges, g_up / g_down slices) and, with
    all experts, the output and dx of ``n_tokens`` sampled tokens; routing, permutation and counts are checked
    for every token."""
    r = _run_block(dev, T, d, E, K, F, seed=seed, experts=picks)
    ref, slot = r["ref"], r["slot"]
    assert torch.equal(slot.chosen_experts.cpu(), ref["ids"])
    assert torch.equal(slot.index_mapping.cpu(), ref["mapping"])
    assert torch.equal(slot.expert_counts.cpu(), ref["counts"])
    off = o_moe.expert_offsets(ref["counts"])
    for e in picks:
        a, b = int(off[e]), int(off[e + 1])
        _close_scaled(slot.x_up[a:b], ref["pre"][a:b], f"x_up rows of expert {e}")
        _close_scaled(r["grads"]["g_up"][e], ref["g_up"][e], f"g_up[{e}]")
        _close_scaled(r["grads"]["g_down"][e], ref["g_down"][e], f"g_down[{e}]")
    # out and dx at full size: every token's rows are independent of the other tokens' (the grouped
    # buffers only reorder them; tests/test_oracle_moe.py pins that property of the oracle), so the
    # oracle runs the whole block, all experts, on a sample of tokens with the GPU's own logits
    g = gen(77)
    tok = torch.cat([torch.tensor([0, 1, T // 2 - 1, T // 2, T - 2, T - 1]), torch.randint(0, T, (n_tokens - 6,), generator=g)])
    xs, ws = r["x"], r["weights_cpu"]
    small = o_moe.routed_block_fwd_bwd(xs[tok], slot.x_router.cpu()[tok], ws["w_router"], ws["w_up"], ws["w_down"],
                                       r["res"][tok], r["dy"][tok], K)
    assert torch.equal(small["ids"], ref["ids"][tok])
    _close_scaled(r["out"].cpu()[tok], small["out"], "out of the sampled tokens")
    _close_scaled(r["dx"].cpu()[tok], small["dx"], "dx of the sampled tokens")
    assert torch.isfinite(r["out"].float()).all() and torch.isfinite(r["dx"].float()).all()
    assert int(slot.expert_counts.sum()) == T * K


def test_block_full_size_qwen3_30b_a3b(dev):
    """8192 tokens, hidden 2048, 128 experts, top-8, intermediate 768."""
    _check_sampled_block(dev, 8192, 2048, 128, 8, 768, picks=(0, 1, 31, 64, 100, 127), seed=1004)


def test_block_reference_parity_shape(dev):
    """The shape the reference quotes for its own backend parity gate (tests/moe/README.md:262-264):
    T = 2048, top-8 of 256 experts, intermediate 1024, hidden 2048 (64 rows per expert on average:
    128-row tiles, many experts with few rows)."""
    _check_sampled_block(dev, 2048, 2048, 256, 8, 1024, picks=(0, 1, 2, 77, 128, 200, 254, 255), seed=1005, n_tokens=24)


def test_recompute_and_phase_ops(dev):
    g = gen(11)
    T, d, E, K, F = 256, 128, 8, 2, 64
    x = randn(g, T, d).to(dev)
    w_up = randn(g, E, 2 * F, d, std=0.05).to(dev)
    w_down = randn(g, E, d, F, std=0.05).to(dev)
    w_router = randn(g, d, E, std=0.05).to(dev)
    slot = _slot(T, K, E, F, torch.bfloat16, dev)
    stream = torch.cuda.current_stream()
    rw, ids = full_moe.route_topk_softmax(x, w_router, top_k=K, routing_mode="topk_then_softmax",
                                          gate_logits_out=slot.x_router, topk_ids_out=slot.chosen_experts,
                                          topk_weights_out=slot.router_weights)
    host = torch.zeros(E, dtype=torch.int32).pin_memory()
    sx = torch.empty(T * K, d, dtype=torch.bfloat16, device=dev)
    idx, host2 = full_moe.dispatch_scatter(x, rw, ids, num_experts=E, index_mapping=slot.index_mapping,
                                           expert_counts_gpu=slot.expert_counts, expert_counts_cpu=host,
                                           scattered_x_out=sx, scattered_router_weights_out=slot.scattered_router_weights)
    assert host2 is host and int(host.sum()) == T * K      # readable on return (sync=True default)
    # pageable host counts and no device counts buffer lent: the sort's own counts are copied
    pageable = torch.zeros(E, dtype=torch.int32)
    sx2 = torch.empty_like(sx)
    srw2 = torch.empty_like(slot.scattered_router_weights)
    idx2, host3 = full_moe.dispatch_scatter(x, rw, ids, num_experts=E, index_mapping=None, expert_counts_gpu=None,
                                            expert_counts_cpu=pageable, scattered_x_out=sx2,
                                            scattered_router_weights_out=srw2)
    assert host3 is pageable and torch.equal(pageable, host) and torch.equal(idx2, idx) and torch.equal(sx2, sx)
    saved = sx.clone()
    full_moe.swiglu_expert_loop_fwd(sx, slot.x_up, w_up, w_down, host, primary_stream=stream, secondary_stream=None,
                                    x_act_even=None, x_act_odd=None)
    pre = slot.x_up.clone()
    slot.x_up.zero_()
    backend = FlextrainMoEExpertCompute()
    handoff = backend.fwd_recompute(x, dict(w_up=w_up, w_down=w_down), slot=slot,
                                    chunk_extra={backend._CHUNK_EXTRA_HOST_COUNTS: {0: host}}, layer_id=0,
                                    primary_stream=stream, secondary_stream=None,
                                    scratch_fn=lambda s, dt: torch.empty(s, dtype=dt, device=dev))
    assert torch.equal(handoff, saved) and torch.equal(slot.x_up, pre)


@pytest.mark.parametrize("E,TK", [(8, 1000), (3, 5000)])
def test_one_plan_serves_every_grouped_launch_of_a_routing(dev, E, TK):
    """A GroupedPlan made once from the counts gives the same bits as each launch planning for itself."""
    from flextrain_amd.ops.grouped import GroupedPlan, flextrain_grouped_gemm_rows_glu

    g = gen(E + TK)
    K, F = 128, 96
    counts = _ragged_counts(g, E, TK).to(dev)
    A = randn(g, TK, K, std=0.5).to(dev)
    W = randn(g, E, 2 * F, K, std=0.1).to(dev)
    Bw = randn(g, TK, 2 * F, std=0.5).to(dev)
    plan = GroupedPlan(counts, E, TK, dev)
    D0, D1 = (torch.full((TK, 2 * F), 7.0, dtype=torch.bfloat16, device=dev) for _ in range(2))
    flextrain_grouped_gemm_rows(A, W.transpose(1, 2), counts, D0)
    flextrain_grouped_gemm_rows(A, W.transpose(1, 2), None, D1, plan=plan)
    assert torch.equal(D0, D1)
    G0 = randn(g, E, K, 2 * F).to(dev)
    G1 = G0.clone()
    flextrain_grouped_gemm_wgrad(A, Bw, G0, counts)
    flextrain_grouped_gemm_wgrad(A, Bw, G1, None, plan=plan)
    assert torch.equal(G0, G1)
    pre0, pre1 = torch.empty_like(D0), torch.empty_like(D0)
    act0, act1 = (torch.empty(TK, F, dtype=torch.bfloat16, device=dev) for _ in range(2))
    flextrain_grouped_gemm_rows_glu(A, W, counts, pre0, act0)
    flextrain_grouped_gemm_rows_glu(A, W, None, pre1, act1, plan=plan)
    assert torch.equal(pre0, pre1) and torch.equal(act0, act1)
    with pytest.raises(ValueError):
        flextrain_grouped_gemm_rows(A[:10], W.transpose(1, 2), None, D1[:10], plan=plan)


def test_walking_kernels_fp16_and_int64_row_sources(dev):
    """fp16 through the 256-row walking kernels (rows form and weight gradient), and the row map from an
    int64 index mapping."""
    from flextrain_amd.ops import moe as moe_ops

    g = gen(4242)
    E, TK, K, N = 3, 2400, 160, 264          # 800 rows per expert on average: 256-row tiles, K tail of 32
    counts = _ragged_counts(g, E, TK)
    A = randn(g, TK, K, std=0.5, dtype=torch.float16)
    W = randn(g, E, N, K, std=0.1, dtype=torch.float16)
    D = torch.empty(TK, N, dtype=torch.float16, device=dev)
    flextrain_grouped_gemm_rows(A.to(dev), W.to(dev).transpose(1, 2), counts.to(dev), D)
    off = o_moe.expert_offsets(counts)
    for e in range(E):
        a, b = int(off[e]), int(off[e + 1])
        if a < b:
            _close_scaled(D[a:b], A[a:b].float() @ W[e].float().t(), f"rows, expert {e}")
    B = randn(g, TK, N, std=0.5, dtype=torch.float16)
    G0 = randn(g, E, K, N, dtype=torch.float16)
    G = G0.to(dev).clone()
    flextrain_grouped_gemm_wgrad(A.to(dev), B.to(dev), G, counts.to(dev))
    for e in range(E):
        a, b = int(off[e]), int(off[e + 1])
        _close_scaled(G[e], G0[e].float() + A[a:b].float().t() @ B[a:b].float(), f"wgrad, expert {e}")
    ids = torch.stack([torch.randperm(8, generator=g)[:2] for _ in range(50)]).to(torch.int64).to(dev)
    mapping, _ = moe_ops.flextrain_moe_sort(ids, num_experts=8)
    src32 = moe_ops.flextrain_moe_row_sources(mapping.to(torch.int32))
    src64 = moe_ops.flextrain_moe_row_sources(mapping.to(torch.int64))
    assert torch.equal(src32, src64)


def test_stale_or_foreign_plan_is_not_consumed(dev):
    """A grouped launch given no counts takes the plan in its workspace.  Through the raw C ABI: a
    workspace that was never planned, and one planned for another expert count, leave the output
    untouched instead of sending the kernel through garbage tile lists; a gathered up-projection whose
    row map holds out-of-range entries stays inside the source matrix."""
    from flextrain_amd._lib import dtype_enum, lib, ptr, stream_ptr
    from flextrain_amd.ops.grouped import GroupedPlan, flextrain_grouped_gemm_rows_glu

    g = gen(808)
    E, TK, K, N = 4, 2400, 128, 256           # 600 rows per expert: the walking 256-row kernels
    counts = torch.full((E,), TK // E, dtype=torch.int32, device=dev)
    A = randn(g, TK, K, std=0.5).to(dev)
    W = randn(g, E, N, K, std=0.1).to(dev)
    L = lib()
    nbytes = int(L.fx_grouped_ws_bytes(E, TK))

    def raw_rows(ws, counts_ptr, D):
        rc = L.fx_grouped_gemm_rows(ptr(A), K, ptr(W), K, N * K, 1, None, 0, ptr(D), N, counts_ptr, E, TK, N, K, 1.0, 0.0,
                                    dtype_enum(torch.bfloat16), ptr(ws), nbytes, stream_ptr(dev))
        assert rc == 0
        torch.cuda.synchronize()

    want = torch.empty(TK, N, dtype=torch.bfloat16, device=dev)
    ws_good = torch.zeros(nbytes // 4, dtype=torch.int32, device=dev)
    raw_rows(ws_good, counts.data_ptr(), want)
    again = torch.full_like(want, 7.0)
    raw_rows(ws_good, None, again)                        # the plan the first call left: same bits
    assert torch.equal(again, want)
    for ws in (torch.zeros(nbytes // 4, dtype=torch.int32, device=dev),
               torch.full((nbytes // 4,), 0x7fffffff, dtype=torch.int32, device=dev),
               GroupedPlan(torch.full((E + 1,), 100, dtype=torch.int32, device=dev), E + 1, TK, dev).ws[:nbytes // 4].clone()):
        D = torch.full((TK, N), 7.0, dtype=torch.bfloat16, device=dev)
        raw_rows(ws, None, D)
        assert bool((D == 7.0).all())
    # row map with entries outside [0, rows of x): clamped, finite results, rows with valid entries exact
    T, F = 300, 64
    x = randn(g, T, K, std=0.5).to(dev)
    Wg = randn(g, E, 2 * F, K, std=0.1).to(dev)
    src = torch.randint(0, T, (TK,), generator=g).to(torch.int32)
    src[::7] = 1 << 30
    src[3::11] = -5
    pre = torch.empty(TK, 2 * F, dtype=torch.bfloat16, device=dev)
    act = torch.empty(TK, F, dtype=torch.bfloat16, device=dev)
    flextrain_grouped_gemm_rows_glu(x, Wg, counts, pre, act, row_sources=src.to(dev))
    clamped = src.clamp(0, T - 1).long()
    pre2, act2 = torch.empty_like(pre), torch.empty_like(act)
    flextrain_grouped_gemm_rows_glu(x, Wg, counts, pre2, act2, row_sources=clamped.to(torch.int32).to(dev))
    assert torch.equal(pre, pre2) and torch.equal(act, act2) and bool(torch.isfinite(pre.float()).all())


@pytest.mark.parametrize("E,TK,d,F", [(4, 2400, 128, 64), (3, 1800, 256, 264), (128, 65536, 2048, 768)])
@pytest.mark.parametrize("dprob_dtype", [torch.bfloat16, torch.float32])
def test_fused_dgrad_swiglu_bwd_equals_the_two_launches(dev, E, TK, d, F, dprob_dtype):
    """Steps (a) + (b) of the expert backward (flextrain/ops/full_moe.py:589-600) as one launch against
    the dgrad GEMM followed by the SwiGLU-backward kernel: dx_up and the saved activation bit for bit
    (both evaluate the same element function on the same rounded dx_act), the router-weight gradient
    within the bf16 tolerance (its fp32 row sum runs in another order), and against the oracle."""
    from flextrain_amd.ops import moe as moe_ops
    from flextrain_amd.ops.grouped import (flextrain_grouped_gemm_rows_swiglu_bwd, grouped_swiglu_bwd_supported)

    g = gen(E * 31 + F)
    counts = _ragged_counts(g, E, TK)
    dy = randn(g, TK, d, std=0.5)
    w_down = randn(g, E, d, F, std=0.1)
    x_up = randn(g, TK, 2 * F)
    srw = torch.rand(TK, 1, generator=g).to(torch.bfloat16)
    dyd, wd, xd, sd, cd = dy.to(dev), w_down.to(dev), x_up.to(dev), srw.to(dev), counts.to(dev)
    # the two launches
    dx_act = torch.empty(TK, F, dtype=torch.bfloat16, device=dev)
    flextrain_grouped_gemm_rows(dyd, wd, cd, dx_act)
    dx_ref = torch.empty(TK, 2 * F, dtype=torch.bfloat16, device=dev)
    act_ref = torch.empty(TK, F, dtype=torch.bfloat16, device=dev)
    dw_ref = torch.empty(TK, 1, dtype=dprob_dtype, device=dev)
    moe_ops.flextrain_swiglu_moe_bwd(dx_act, xd, sd, dx=dx_ref, dw=dw_ref, fwd_act=act_ref)
    # one launch
    dx = torch.full_like(dx_ref, 7.0)
    act = torch.full_like(act_ref, 7.0)
    dw = torch.full_like(dw_ref, 7.0)
    assert grouped_swiglu_bwd_supported(dyd, wd, xd, sd, dx, act, dw)
    flextrain_grouped_gemm_rows_swiglu_bwd(dyd, wd, cd, xd, sd, dx, dw, fwd_act=act)
    assert torch.equal(dx, dx_ref), f"dx_up differs in {int((dx != dx_ref).sum())} of {dx.numel()} elements"
    assert torch.equal(act, act_ref)
    _close_scaled(dw, dw_ref, "router-weight gradient, fused vs two launches")
    # twice the same bits (fixed summation order)
    dw2 = torch.empty_like(dw)
    flextrain_grouped_gemm_rows_swiglu_bwd(dyd, wd, cd, xd, sd, torch.empty_like(dx), dw2, fwd_act=None)
    assert torch.equal(dw, dw2)
    # against the oracle on a few experts
    off = o_moe.expert_offsets(counts)
    for e in (range(E) if E <= 8 else (0, 2, 127)):
        a, b = int(off[e]), int(off[e + 1])
        if a == b:
            continue
        dact = (dy[a:b].float() @ w_down[e].float()).to(torch.bfloat16)
        want_dx, want_dw, want_act = o_moe.swiglu_moe_bwd(dact, x_up[a:b], srw[a:b])
        _close_scaled(dx[a:b], want_dx, f"dx_up of expert {e}")
        _close_scaled(act[a:b], want_act, f"saved activation of expert {e}")
        _close_scaled(dw[a:b].reshape(-1), want_dw.reshape(-1), f"router-weight gradient of expert {e}")


@pytest.mark.parametrize("T,E,K,d,F", [(1200, 4, 2, 192, 136), (1200, 4, 2, 200, 136), (8192, 128, 8, 2048, 768)])
def test_backward_launches_gather_unsorted_rows_bit_for_bit(dev, T, E, K, d, F):
    """The expert backward without expert-sorted copies of dy and x: the fused dgrad launch (rows of
    the unsorted upstream gradient through the row map) and both weight-gradient launches (unsorted
    operand gathered along the contraction, as A and as B) against the same launches on the scattered
    copies.  Same values reach the same MFMAs in the same order: every output must match bit for bit."""
    from flextrain_amd.ops import moe as moe_ops
    from flextrain_amd.ops.grouped import flextrain_grouped_gemm_rows_swiglu_bwd

    g = gen(T + E)
    TK = T * K
    logits = torch.randn(T, E, generator=g)
    ids = logits.topk(K, dim=1).indices.to(torch.int32).to(dev)
    mapping, counts = moe_ops.flextrain_moe_sort(ids, num_experts=E)
    src = moe_ops.flextrain_moe_row_sources(mapping)
    dy, x = randn(g, T, d, std=0.5).to(dev), randn(g, T, d, std=0.5).to(dev)
    sdy, sx = torch.empty(TK, d, dtype=torch.bfloat16, device=dev), torch.empty(TK, d, dtype=torch.bfloat16, device=dev)
    moe_ops.flextrain_moe_scatter(dy, mapping, out=sdy)
    moe_ops.flextrain_moe_scatter(x, mapping, out=sx)
    w_down = randn(g, E, d, F, std=0.1).to(dev)
    x_up = randn(g, TK, 2 * F).to(dev)
    srw = torch.rand(TK, 1, generator=g).to(torch.bfloat16).to(dev)

    def fused(dy_arg, rows):
        dx = torch.full((TK, 2 * F), 7.0, dtype=torch.bfloat16, device=dev)
        act = torch.full((TK, F), 7.0, dtype=torch.bfloat16, device=dev)
        dw = torch.full((TK, 1), 7.0, dtype=torch.bfloat16, device=dev)
        flextrain_grouped_gemm_rows_swiglu_bwd(dy_arg, w_down, counts, x_up, srw, dx, dw, fwd_act=act, row_sources=rows)
        return dx, act, dw

    for got, want, what in zip(fused(dy, src), fused(sdy, None), ("dx_up", "saved activation", "router-weight gradient")):
        assert torch.equal(got, want), f"{what}: {int((got != want).sum())} of {got.numel()} elements differ"
    dx_up = fused(sdy, None)[0]
    act = fused(sdy, None)[1]
    for gdt in (torch.bfloat16, torch.float32):
        g0 = randn(g, E, d, F, dtype=gdt).to(dev)
        ga, gb = g0.clone(), g0.clone()
        flextrain_grouped_gemm_wgrad(sdy, act, ga, counts)                              # g_down, sorted A
        flextrain_grouped_gemm_wgrad(dy, act, gb, counts, a_row_sources=src)            # g_down, gathered A
        assert torch.equal(ga, gb), f"g_down ({gdt}): {int((ga != gb).sum())} elements differ"
        g1 = randn(g, E, 2 * F, d, dtype=gdt).to(dev)
        ga, gb = g1.clone(), g1.clone()
        flextrain_grouped_gemm_wgrad(dx_up, sx, ga, counts)                             # g_up, sorted B
        flextrain_grouped_gemm_wgrad(dx_up, x, gb, counts, b_row_sources=src)           # g_up, gathered B
        assert torch.equal(ga, gb), f"g_up ({gdt}): {int((ga != gb).sum())} elements differ"
    # a map with entries outside the source is clamped, never followed out of bounds
    bad = src.clone()
    bad[::5] = 1 << 30
    bad[1::7] = -3
    gc, gd = g1.clone(), g1.clone()
    flextrain_grouped_gemm_wgrad(dx_up, x, gc, counts, b_row_sources=bad)
    flextrain_grouped_gemm_wgrad(dx_up, x, gd, counts, b_row_sources=bad.clamp(0, T - 1))
    assert torch.equal(gc, gd) and bool(torch.isfinite(gc.float()).all())
    with pytest.raises(ValueError):
        flextrain_grouped_gemm_wgrad(dy, x, g1, counts, a_row_sources=src, b_row_sources=src)
