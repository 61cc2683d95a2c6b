"""GEMM dispatcher with the interface of the reference's ``matmul_dispatcher``
package (helpers/matmul_dispatcher/matmul_dispatcher/__init__.py:63-276):
``D = alpha * A @ B + beta * C`` on strided row-major / column-major 2-D
tensors, fp32 accumulation, explicit stream pointer.

``CublasLtDispatcher`` is kept as the class name callers import; it drives the
hand-written MFMA GEMM of libflexhip.so through ``dispatch_matmul``.  The 64 MiB
workspace of the reference class is kept (split-K partial sums live there) but is
allocated on the first call, so nothing touches the GPU at import or construction
time.
"""
from __future__ import annotations

import ctypes
import time

import torch

from ._lib import lib

_dtype_to_enum = {torch.float16: 1, torch.bfloat16: 2, torch.float32: 0}


def _get_layout(t):
    """``(data_ptr, leading_dim, trans_flag)``: unit column stride -> row-major
    (trans 0, ld = row stride); unit row stride -> column-major (trans 1,
    ld = column stride).  helpers/matmul_dispatcher/matmul_dispatcher/__init__.py:63-90."""
    if t.dim() != 2:
        raise ValueError("Only 2D tensors supported for matmul dispatcher.")
    stride_row, stride_col = t.stride()
    if stride_col == 1:
        return t.data_ptr(), stride_row, 0
    if stride_row == 1:
        return t.data_ptr(), stride_col, 1
    raise ValueError(
        f"Tensor memory layout not supported (Strides: {t.stride()}). "
        "Must be Row-Major (stride[:,-1]==1) or Col-Major (stride[:,0]==1).")


def tensor_layout(t):
    """Return ``(data_ptr, leading_dim, trans_flag)`` for a 2-D tensor."""
    return _get_layout(t)


def dtype_enum(dtype):
    """torch dtype -> 0 fp32 / 1 fp16 / 2 bf16."""
    try:
        return _dtype_to_enum[dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {dtype} for matmul_fast") from None


_fast_entry = None


def _bind_fast():
    """The C fast-call entry (``flextrain_amd/csrc/pyext/dispatch_fast.c``), bound to the
    ``dispatch_matmul`` of the library this process has loaded.  Raises when the extension has
    not been built: there is no slower stand-in behind it."""
    global _fast_entry
    if _fast_entry is None:
        from . import _dispatch_fast      # ImportError when the extension is missing
        _dispatch_fast.bind(ctypes.cast(lib().dispatch_matmul, ctypes.c_void_p).value)
        _fast_entry = _dispatch_fast.matmul_fast
    return _fast_entry


def matmul_fast(*args):
    """Raw 24-argument entry with the argument order and error behaviour of the reference's
    ``matmul_fast`` (helpers/matmul_dispatcher/src/dispatch_pyext.cpp:37-140): ``TypeError`` for any
    other argument count, ``RuntimeError`` when ``dispatch_matmul`` reports failure.  After the first
    call the module attribute IS the C function (no Python frame in between)."""
    global matmul_fast
    matmul_fast = _bind_fast()
    return matmul_fast(*args)


class CublasLtDispatcher:
    """Same constructor and methods as the reference class of this name
    (helpers/matmul_dispatcher/matmul_dispatcher/__init__.py:125-276)."""

    def __init__(self, round_multiple=32, max_algos=5):
        self.round_multiple = round_multiple
        self.max_algos = max_algos
        self._lib = lib()
        self.ctx = self._lib.create_dispatcher(round_multiple, max_algos)
        self.workspace_size = 64 * 1024 * 1024
        self.workspace = None           # allocated on first use, on the device of the first operand
        self.ws_ptr = 0
        self.fp16 = torch.float16
        self.bf16 = torch.bfloat16
        self.total_python_ns = 0
        self._ctx_int = int(self.ctx) if self.ctx is not None else 0
        self._fast = self._bind_on_first_fast_call   # ``matmul`` (ctypes) works without the C extension

    def _bind_on_first_fast_call(self, *args):
        """Stands in for the C entry until it is first needed; from then on ``self._fast`` IS the C
        function.  A missing extension is reported here, where it is needed, and not by the constructor."""
        try:
            self._fast = _bind_fast()
        except ImportError as err:
            raise ImportError("flextrain_amd._dispatch_fast is not built for this interpreter "
                              "(make -C flextrain_amd/csrc PYTHON=<this python>); the validating "
                              "matmul() path does not need it") from err
        return self._fast(*args)

    def __del__(self):
        if getattr(self, "ctx", None):
            self._lib.destroy_dispatcher(self.ctx)
            self.ctx = None

    def _ensure_workspace(self, device):
        if self.workspace is None or self.workspace.device != device:
            self.workspace = torch.empty(self.workspace_size, dtype=torch.uint8, device=device)
            self.ws_ptr = self.workspace.data_ptr()

    def get_stats(self):
        stats = (ctypes.c_uint64 * 7)()
        self._lib.get_stats(self.ctx, stats)
        calls = stats[1]
        if calls == 0:
            return {"matmuls_called": 0, "algos_saved": 0, "algo_hits": 0, "avg_wrapper_overhead_us": 0,
                    "avg_cpp_total_us": 0, "breakdown": {"driver_submit_us": 0, "cpp_hash_logic_us": 0}}
        total_cpp_ns, total_driver_ns = stats[3], stats[6]
        return {
            "matmuls_called": calls,
            "algos_saved": stats[0],
            "algo_hits": stats[2],
            "avg_wrapper_overhead_us": (self.total_python_ns / calls / 1000.0) - (total_cpp_ns / calls / 1000.0),
            "avg_cpp_total_us": total_cpp_ns / calls / 1000.0,
            "breakdown": {"driver_submit_us": total_driver_ns / calls / 1000.0,
                          "cpp_hash_logic_us": (total_cpp_ns - total_driver_ns) / calls / 1000.0},
        }

    def matmul(self, stream_ptr, A, B, C=None, D=None, alpha=1.0, beta=0.0):
        """``D = alpha * A @ B + beta * C``; allocates ``D`` when it is None."""
        t0 = time.perf_counter_ns()
        ptr_A, ld_A, trans_a = _get_layout(A)
        ptr_B, ld_B, trans_b = _get_layout(B)
        M, K = A.shape
        K_B, N = B.shape
        if K != K_B:
            raise ValueError(f"Shape Mismatch: A is {A.shape}, B is {B.shape}. Inner dims {K} vs {K_B} must match.")
        if D is None:
            D = torch.empty((M, N), dtype=A.dtype, device=A.device)
        ptr_D, ld_D, trans_d = _get_layout(D)
        if trans_d != 0:
            raise ValueError("Output tensor D must be Row-Major for this dispatcher.")
        if C is not None:
            ptr_C, ld_C, trans_c = _get_layout(C)
            if trans_c != 0:
                raise ValueError("Bias/Add tensor C must be Row-Major.")
        else:
            ptr_C, ld_C = 0, N
        if M == 0 or N == 0 or K == 0:
            raise ValueError(f"All dimensions must be non-zero. Got M={M}, N={N}, K={K}")
        dt = 1 if A.dtype == self.fp16 else (2 if A.dtype == self.bf16 else 0)
        d_dt = _dtype_to_enum.get(D.dtype, dt)
        self._ensure_workspace(A.device)
        ret = self._lib.dispatch_matmul(self.ctx, stream_ptr, M, N, K, ptr_A, ld_A, ptr_B, ld_B, ptr_C, ld_C,
                                        ptr_D, ld_D, self.ws_ptr, self.workspace_size, dt, dt, d_dt, d_dt, 0,
                                        alpha, beta, trans_a, trans_b)
        if ret != 0:
            raise RuntimeError("Failed to dispatch matmul")
        self.total_python_ns += time.perf_counter_ns() - t0
        return D

    def matmul_shared_a(self, stream_ptr, A, Bs, Ds, Cs=None, alpha=1.0, beta=0.0):
        """``Ds[i] = alpha * A @ Bs[i] + beta * Cs[i]`` for up to four ``Bs`` in ONE launch when the
        operands allow it (bf16 / fp16, outputs of the input type, every ``B`` in the same
        row- or column-major form, 16-byte aligned with multiples of 8 on the contiguous axes);
        otherwise one :meth:`matmul` per product.  Same results either way.  No counterpart in
        the reference, which calls ``matmul`` once per projection (attention.py:424-463): products
        like the key / value projections are each too small to fill the GPU alone."""
        n = len(Bs)
        if len(Ds) != n or (Cs is not None and len(Cs) != n):
            raise ValueError("matmul_shared_a: Bs, Ds and Cs must have the same length")
        if self._segments_ok(A, Bs, Ds, Cs):
            ptr_A, ld_A, trans_a = _get_layout(A)
            lays = [_get_layout(b) for b in Bs]
            M, K = A.shape
            vp, i64 = ctypes.c_void_p * n, ctypes.c_int64 * n
            b_ptrs, b_ld = vp(*[l[0] for l in lays]), i64(*[l[1] for l in lays])
            d_ptrs, d_ld = vp(*[d.data_ptr() for d in Ds]), i64(*[d.stride(0) for d in Ds])
            if Cs is not None and beta != 0.0:
                c_ptrs, c_ld = vp(*[c.data_ptr() for c in Cs]), i64(*[c.stride(0) for c in Cs])
            else:
                c_ptrs, c_ld = None, None
            ns = (ctypes.c_int * n)(*[b.shape[1] for b in Bs])
            rc = self._lib.fx_gemm_segments(ptr_A, ld_A, trans_a, n, b_ptrs, b_ld, lays[0][2], c_ptrs, c_ld, d_ptrs,
                                            d_ld, M, ns, K, alpha, beta, _dtype_to_enum[A.dtype], stream_ptr)
            if rc != 0:
                raise RuntimeError("fx_gemm_segments failed")
            return Ds
        for i in range(n):
            self.matmul(stream_ptr, A, Bs[i], C=None if Cs is None else Cs[i], D=Ds[i], alpha=alpha, beta=beta)
        return Ds

    @staticmethod
    def _segments_ok(A, Bs, Ds, Cs):
        if not 2 <= len(Bs) <= 4 or A.dim() != 2 or A.dtype not in (torch.bfloat16, torch.float16):
            return False
        M, K = A.shape
        if M == 0 or K == 0:
            return False

        def operand_ok(t, rows, cols):
            if t.dim() != 2 or t.shape[0] != rows or t.dtype != A.dtype or t.data_ptr() % 16:
                return False
            sr, sc = t.stride()
            if sc == 1:      # row-major: the columns are contiguous
                return sr % 8 == 0 and sr < (1 << 23) and (cols is None or cols % 8 == 0) and t.shape[1] % 8 == 0
            if sr == 1:      # column-major: the rows are contiguous
                return sc % 8 == 0 and sc < (1 << 23) and rows % 8 == 0
            return False

        if not operand_ok(A, M, None):
            return False
        form = None
        for i, b in enumerate(Bs):
            if not operand_ok(b, K, None) or b.shape[1] <= 0:
                return False
            f = b.stride(1) == 1
            if form is None:
                form = f
            if f != form:
                return False
            d = Ds[i]
            if d.dim() != 2 or d.shape != (M, b.shape[1]) or d.dtype != A.dtype or d.stride(1) != 1:
                return False
            if Cs is not None:
                c = Cs[i]
                if c.dim() != 2 or c.shape != d.shape or c.dtype != A.dtype or c.stride(1) != 1:
                    return False
        return True

    def matmul_sum(self, stream_ptr, As, Bs, C=None, D=None, alpha=1.0, beta=0.0):
        """``D = alpha * sum_i As[i] @ Bs[i] + beta * C`` for up to four products in ONE launch when
        the operands allow it (bf16 / fp16; every ``A`` in one form and every ``B`` in one form;
        16-byte aligned with multiples of 8 on K, the contiguous axes and the leading dimensions):
        the sum is formed in fp32 and rounded once.  Otherwise one :meth:`matmul` per product,
        accumulating through ``D`` (rounded after each, as the reference's chains of ``beta = 1``
        calls are: attention.py:712-775, ffn_dense.py:193-235)."""
        n = len(As)
        if n == 0 or len(Bs) != n:
            raise ValueError("matmul_sum: As and Bs must be non-empty and of the same length")
        M, N = As[0].shape[0], Bs[0].shape[1]
        if D is None:
            D = torch.empty((M, N), dtype=As[0].dtype, device=As[0].device)
        if self._ksum_ok(As, Bs, C, D):
            la, lb = [_get_layout(a) for a in As], [_get_layout(b) for b in Bs]
            vp, i64 = ctypes.c_void_p * n, ctypes.c_int64 * n
            ks = (ctypes.c_int * n)(*[a.shape[1] for a in As])
            use_c = C is not None and beta != 0.0
            rc = self._lib.fx_gemm_ksum(n, vp(*[l[0] for l in la]), i64(*[l[1] for l in la]), la[0][2],
                                        vp(*[l[0] for l in lb]), i64(*[l[1] for l in lb]), lb[0][2], ks,
                                        C.data_ptr() if use_c else None, C.stride(0) if use_c else 0, D.data_ptr(),
                                        D.stride(0), M, N, alpha, beta if use_c else 0.0,
                                        _dtype_to_enum[As[0].dtype], _dtype_to_enum[D.dtype], stream_ptr)
            if rc != 0:
                raise RuntimeError("fx_gemm_ksum failed")
            return D
        self.matmul(stream_ptr, As[0], Bs[0], C=C, D=D, alpha=alpha, beta=beta)
        for i in range(1, n):
            self.matmul(stream_ptr, As[i], Bs[i], C=D, D=D, alpha=alpha, beta=1.0)
        return D

    @staticmethod
    def _ksum_ok(As, Bs, C, D):
        n = len(As)
        if not 2 <= n <= 4:
            return False
        dt = As[0].dtype
        if dt not in (torch.bfloat16, torch.float16) or As[0].dim() != 2 or Bs[0].dim() != 2:
            return False
        M, N = As[0].shape[0], Bs[0].shape[1]
        if M == 0 or N == 0:
            return False
        if D.dim() != 2 or D.shape != (M, N) or D.stride(1) != 1 or not (D.dtype == dt or (dt == torch.bfloat16 and D.dtype == torch.float32)):
            return False
        if C is not None and (C.dim() != 2 or C.shape != (M, N) or C.stride(1) != 1 or C.dtype != D.dtype):
            return False

        def form(t):     # 0 row-major, 1 column-major, None unsupported
            if t.dim() != 2 or t.dtype != dt or t.data_ptr() % 16:
                return None
            sr, sc = t.stride()
            if sc == 1 and sr % 8 == 0 and sr < (1 << 23) and t.shape[1] % 8 == 0:
                return 0
            if sr == 1 and sc % 8 == 0 and sc < (1 << 23) and t.shape[0] % 8 == 0:
                return 1
            return None

        fa, fb = form(As[0]), form(Bs[0])
        if fa is None or fb is None:
            return False
        for a, b in zip(As, Bs):
            K = a.shape[1]
            if a.shape[0] != M or b.shape != (K, N) or K == 0 or K % 8 or form(a) != fa or form(b) != fb:
                return False
        return True

    def matmul_fast(self, stream_ptr, A, B, C=None, D=None, alpha=1.0, beta=0.0):
        """Hot-path variant: no validation, no allocation (``D`` required), no
        wrapper timing.  Bit-identical results to :meth:`matmul`."""
        a_stride = A.stride()
        if a_stride[1] == 1:
            ptr_A, ld_A, trans_a = A.data_ptr(), a_stride[0], 0
        else:
            ptr_A, ld_A, trans_a = A.data_ptr(), a_stride[1], 1
        b_stride = B.stride()
        if b_stride[1] == 1:
            ptr_B, ld_B, trans_b = B.data_ptr(), b_stride[0], 0
        else:
            ptr_B, ld_B, trans_b = B.data_ptr(), b_stride[1], 1
        ptr_D, ld_D = D.data_ptr(), D.stride(0)
        if C is None:
            ptr_C, ld_C = 0, ld_D
        else:
            ptr_C, ld_C = C.data_ptr(), C.stride(0)
        M, K = A.shape
        _, N = B.shape
        dt = _dtype_to_enum[A.dtype]
        d_dt = _dtype_to_enum[D.dtype]
        if self.workspace is None:
            self._ensure_workspace(A.device)
        self._fast(self._ctx_int, stream_ptr, M, N, K, ptr_A, ld_A, trans_a, ptr_B, ld_B, trans_b, ptr_C, ld_C,
                   ptr_D, ld_D, self.ws_ptr, self.workspace_size, dt, dt, d_dt, d_dt, 0, alpha, beta)
        return D
