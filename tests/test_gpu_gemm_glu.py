"""GEMMs with the gated activation in the epilogue against the separate launches they replace
(pre-activations bit-identical; the activation bit-identical where both paths share the device
function) and against the CPU oracle (bf16: rtol = atol = 1e-2)."""
import pytest
import torch

from flextrain_amd import ops
from flextrain_amd.ops.grouped import (
    dual_glu_supported,
    flextrain_gemm_dual_glu,
    flextrain_grouped_gemm_rows,
    flextrain_grouped_gemm_rows_glu,
    grouped_glu_supported,
)
from oracle import glu as o_glu
from util import close, gen, randn

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M,N,K", [(512, 256, 128), (1000, 328, 192), (37, 8, 64), (300, 1160, 256)])
@pytest.mark.parametrize("b_rowmajor", [True, False])
@pytest.mark.parametrize("activation,gate_first", [("silu", True), ("silu", False), ("gelu_tanh", True)])
def test_dual_glu_matches_separate_launches(dev, M, N, K, b_rowmajor, activation, gate_first):
    g = gen(M + N + K)
    A = randn(g, M, K).to(dev)
    if b_rowmajor:
        B1, B2 = randn(g, K, N, std=K ** -0.5).to(dev), randn(g, K, N, std=K ** -0.5).to(dev)
    else:
        B1, B2 = randn(g, N, K, std=K ** -0.5).to(dev).T, randn(g, N, K, std=K ** -0.5).to(dev).T
    P1, P2, act = (torch.empty(M, N, dtype=torch.bfloat16, device=dev) for _ in range(3))
    assert dual_glu_supported(A, B1, B2, P1, P2, act)
    out = flextrain_gemm_dual_glu(A, B1, B2, P1, P2, act, activation=activation, gate_first=gate_first)
    assert out is act
    s = torch.cuda.current_stream().cuda_stream
    R1 = ops.dispatcher.matmul(s, A=A, B=B1)
    R2 = ops.dispatcher.matmul(s, A=A, B=B2)
    assert torch.equal(P1, R1) and torch.equal(P2, R2)
    gate, value = (R1, R2) if gate_first else (R2, R1)
    fwd = ops.flextrain_swiglu_fwd if activation == "silu" else ops.flextrain_gelu_tanh_gated_fwd
    assert torch.equal(act, fwd(gate, value))
    o_fwd = o_glu.swiglu_fwd if activation == "silu" else o_glu.gelu_tanh_gated_fwd
    close(act, o_fwd(gate.cpu(), value.cpu()), what="act vs oracle")
    ref1 = (A.cpu().float() @ B1.cpu().float())
    close(P1, ref1.to(torch.bfloat16), atol=1e-2 * max(1.0, float(ref1.abs().max())), what="P1 vs fp32 matmul")


def test_dual_glu_rejects_unsupported(dev):
    A = torch.zeros(16, 72, dtype=torch.bfloat16, device=dev)          # K not a multiple of 64
    B = torch.zeros(72, 64, dtype=torch.bfloat16, device=dev)
    P = torch.zeros(16, 64, dtype=torch.bfloat16, device=dev)
    assert not dual_glu_supported(A, B, B, P, P, P)
    with pytest.raises(RuntimeError):
        flextrain_gemm_dual_glu(A, B, B, P, P.clone(), P.clone())


@pytest.mark.parametrize("E,F,K,rows", [(4, 96, 128, [130, 0, 77, 300]), (8, 384, 256, [1500] * 8), (3, 8, 64, [1, 2, 3])])
def test_grouped_glu_matches_separate_launches(dev, E, F, K, rows):
    g = gen(E * F + K)
    TK = sum(rows)
    A = randn(g, TK, K).to(dev)
    w_up = randn(g, E, 2 * F, K, std=K ** -0.5).to(dev)
    counts = torch.tensor(rows, dtype=torch.int32, device=dev)
    pre, act = torch.full((TK, 2 * F), 7.0, dtype=torch.bfloat16, device=dev), torch.empty(TK, F, dtype=torch.bfloat16, device=dev)
    assert grouped_glu_supported(A, w_up, pre, act)
    flextrain_grouped_gemm_rows_glu(A, w_up, counts, pre, act)
    ref_pre = torch.empty_like(pre)
    flextrain_grouped_gemm_rows(A, w_up.transpose(1, 2), counts, ref_pre)
    assert torch.equal(pre, ref_pre)
    ref_act = ops.flextrain_swiglu_moe_fwd(ref_pre)
    close(act, ref_act, what="act vs the separate kernel")
    close(act, o_glu.swiglu_fwd(ref_pre[:, F:].cpu(), ref_pre[:, :F].cpu()), what="act vs oracle")


@pytest.mark.parametrize("T,topk,E,F,K", [(96, 2, 4, 96, 128),        # small experts: 128-row tiles, 32-wide K-steps
                                          (2048, 4, 8, 384, 256),     # ~1024 rows per expert: 256-row tiles
                                          (5, 1, 3, 8, 64)])
def test_grouped_glu_gathers_token_rows_in_place(dev, T, topk, E, F, K):
    """The up-projection reading the unsorted activations through the row map equals, bit for bit, the
    same launch on the expert-sorted copy that flextrain_moe_scatter makes."""
    g = gen(T * 3 + E + F)
    x = randn(g, T, K).to(dev)
    ids = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(T)]).to(torch.int32).to(dev)
    mapping, counts = ops.flextrain_moe_sort(ids, num_experts=E)
    TK = T * topk
    w_up = randn(g, E, 2 * F, K, std=K ** -0.5).to(dev)
    sx = ops.flextrain_moe_scatter(x, mapping)
    pre_ref, act_ref = torch.empty(TK, 2 * F, dtype=torch.bfloat16, device=dev), torch.empty(TK, F, dtype=torch.bfloat16, device=dev)
    flextrain_grouped_gemm_rows_glu(sx, w_up, counts, pre_ref, act_ref)
    src = ops.flextrain_moe_row_sources(mapping)
    want_src = torch.empty(TK, dtype=torch.int32)
    want_src[mapping.cpu().flatten().long()] = torch.arange(TK, dtype=torch.int32) // topk
    assert torch.equal(src.cpu(), want_src)
    pre, act = torch.full_like(pre_ref, 7.0), torch.full_like(act_ref, 7.0)
    flextrain_grouped_gemm_rows_glu(x, w_up, counts, pre, act, row_sources=src)
    assert torch.equal(pre, pre_ref) and torch.equal(act, act_ref)
    with pytest.raises(ValueError):
        flextrain_grouped_gemm_rows_glu(x, w_up, counts, pre, act, row_sources=src[:-1])
    if topk > 1:
        with pytest.raises(ValueError):
            flextrain_grouped_gemm_rows_glu(x, w_up, counts, pre, act)      # T rows, TK outputs, no map
