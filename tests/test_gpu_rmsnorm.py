"""HIP RMSNorm (through the C ABI) against the CPU oracle.  bf16 tensors at
rtol = atol = 1e-2; fp32 rstd/dW at rtol 1e-4 (dW atol scaled to its sums)."""
import pytest
import torch

from flextrain_amd import ops
from oracle import rmsnorm as o_norm
from util import BF16_ATOL, BF16_RTOL, close, gen, randn

pytestmark = pytest.mark.gpu

SHAPES = [  # (T, D, head_dim)
    (2048, 4096, None),   # full-size first configuration
    (64, 8192, None), (33, 16384, None), (100, 2048, None), (257, 1024, None),
    (70, 512, None), (19, 256, None), (1000, 128, None), (5, 64, None), (3, 8, None),
    (512, 32 * 128, 128), (300, 8 * 64, 64), (7, 4 * 256, 256),
    (13, 100, None), (9, 20000, None), (6, 12, 4),   # unvectorised path
    (1, 4096, None),
]


def _inputs(seed, T, D, hd, dtype, wdtype):
    g = gen(seed)
    x = randn(g, T, D, dtype=dtype)
    w = randn(g, D if hd is None else hd, dtype=wdtype, std=0.02, mean=1.0)
    dy = randn(g, T, D, dtype=dtype)
    return x, w, dy


@pytest.mark.parametrize("T,D,hd", SHAPES)
@pytest.mark.parametrize("dtype,wdtype", [(torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32)])
def test_fwd_and_recompute(dev, T, D, hd, dtype, wdtype):
    x, w, _ = _inputs(1001, T, D, hd, dtype, wdtype)
    y_ref, rstd_ref = o_norm.rmsnorm_fwd(x, w, 1e-5, hd)
    y, rstd = ops.flextrain_rmsnorm_fwd(x.to(dev), w.to(dev), head_dim=hd, rms_norm_eps=1e-5)
    close(y, y_ref, what="y")
    close(rstd, rstd_ref, rtol=1e-4, atol=0, what="rstd")
    y2 = ops.flextrain_rmsnorm_fwd_recompute(x.to(dev), w.to(dev), rstd, head_dim=hd)
    assert torch.equal(y2, y), "recompute must reproduce the forward bit for bit"


def test_fwd_no_weight_fp32_fp16_and_inplace(dev):
    g = gen(7)
    for dtype in (torch.float32, torch.float16):
        x = randn(g, 50, 1024, dtype=dtype)
        y_ref, rstd_ref = o_norm.rmsnorm_fwd(x, None, 1e-6, None)
        xd = x.to(dev)
        y, rstd = ops.flextrain_rmsnorm_fwd(xd, None, output=xd, rms_norm_eps=1e-6)
        assert y.data_ptr() == xd.data_ptr()
        tol = 1e-5 if dtype == torch.float32 else 1e-2
        close(y, y_ref, rtol=tol, atol=tol, what=f"y {dtype}")
        close(rstd, rstd_ref, rtol=1e-4, atol=0)


def test_fwd_per_head_in_place(dev):
    # q/k-norm call pattern: output is X (flextrain/nn/blocks/attention.py:450-457)
    x, w, _ = _inputs(5, 128, 16 * 128, 128, torch.bfloat16, torch.bfloat16)
    y_ref, _ = o_norm.rmsnorm_fwd(x, w, 1e-5, 128)
    xd = x.to(dev)
    y, _ = ops.flextrain_rmsnorm_fwd(xd, w.to(dev), head_dim=128, output=xd)
    close(y, y_ref)


@pytest.mark.parametrize("T,D,hd", SHAPES)
def test_bwd_engine_pattern(dev, T, D, hd):
    """dX given (accumulate), fp32 dW given (accumulate), y re-materialised:
    the call of flextrain/nn/layers/llama.py:341-350."""
    x, w, dy = _inputs(1002, T, D, hd, torch.bfloat16, torch.bfloat16)
    g = gen(77)
    dx_old = randn(g, T, D)
    dw_old = randn(g, w.numel(), dtype=torch.float32)
    _, rstd = o_norm.rmsnorm_fwd(x, w, 1e-5, hd)
    dx_ref, dw_ref, y_ref = o_norm.rmsnorm_bwd(dy, x, w, rstd, hd, dx_old, dw_old, True)
    dxd, dwd = dx_old.to(dev), dw_old.to(dev)
    dx, dw, y = ops.flextrain_rmsnorm_bwd(dy.to(dev), x.to(dev), w.to(dev), rstd.to(dev), head_dim=hd,
                                          dX=dxd, dW=dwd, recompute_output=True)
    assert dx.data_ptr() == dxd.data_ptr() and dw.data_ptr() == dwd.data_ptr()
    close(dx, dx_ref, what="dx")
    close(y, y_ref, what="y")
    rows = T * (1 if hd is None else D // hd)
    close(dw, dw_ref, rtol=1e-4, atol=1e-4 * max(1.0, rows ** 0.5), what="dw")


def test_bwd_fresh_outputs_and_determinism(dev):
    x, w, dy = _inputs(1003, 2048, 4096, None, torch.bfloat16, torch.bfloat16)
    _, rstd = o_norm.rmsnorm_fwd(x, w, 1e-5, None)
    dx_ref, dw_ref, _ = o_norm.rmsnorm_bwd(dy, x, w, rstd)
    args = (dy.to(dev), x.to(dev), w.to(dev), rstd.to(dev))
    dx, dw, y = ops.flextrain_rmsnorm_bwd(*args)
    assert y is None and dw.dtype == torch.float32
    close(dx, dx_ref)
    close(dw, dw_ref, rtol=1e-4, atol=5e-3)
    dx2, dw2, _ = ops.flextrain_rmsnorm_bwd(*args)
    assert torch.equal(dw, dw2) and torch.equal(dx, dx2)


def test_bwd_bf16_dw_and_no_weight(dev):
    x, w, dy = _inputs(9, 96, 512, None, torch.bfloat16, torch.bfloat16)
    _, rstd = o_norm.rmsnorm_fwd(x, w, 1e-5, None)
    dw_old = randn(gen(3), 512)
    _, dw_ref, _ = o_norm.rmsnorm_bwd(dy, x, w, rstd, dw_old=dw_old)
    dwd = dw_old.to(dev)
    _, dw, _ = ops.flextrain_rmsnorm_bwd(dy.to(dev), x.to(dev), w.to(dev), rstd.to(dev), dW=dwd)
    assert dw.dtype == torch.bfloat16
    close(dw, dw_ref, rtol=2e-2, atol=2e-2)
    dx_ref, none_dw, _ = o_norm.rmsnorm_bwd(dy, x, None, rstd)
    dx, dw2, _ = ops.flextrain_rmsnorm_bwd(dy.to(dev), x.to(dev), None, rstd.to(dev))
    assert dw2 is None and none_dw is None
    close(dx, dx_ref)


def test_errors(dev):
    x = torch.zeros(4, 64, device=dev, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.flextrain_rmsnorm_fwd(x, torch.ones(32, device=dev, dtype=torch.bfloat16))
    with pytest.raises(ValueError):
        ops.flextrain_rmsnorm_fwd(x.t())
    with pytest.raises(ValueError):
        ops.flextrain_rmsnorm_fwd(x, head_dim=48)
    with pytest.raises(ValueError):
        ops.flextrain_rmsnorm_fwd(x, rstd=torch.zeros(4, 2, device=dev))
    # empty input is a no-op
    e = torch.zeros(0, 64, device=dev, dtype=torch.bfloat16)
    y, rstd = ops.flextrain_rmsnorm_fwd(e)
    assert y.shape == (0, 64) and rstd.shape == (0, 1)
