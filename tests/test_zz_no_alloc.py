"""The expert sort for callers that cannot allocate (HIP graph capture, allocation-free serving
loops): ``fx_moe_sort_noalloc`` keeps its scratch in a fixed device array instead of a lent
workspace.  Called through the C ABI and compared with ``fx_moe_sort`` (bit-exact: index mapping
and counts are integers), on two calls in a row, the second with a smaller input, so that what
the first call left in the shared array cannot leak into the second."""
import ctypes

import pytest
import torch

from flextrain_amd._lib import lib
from util import gen

pytestmark = pytest.mark.gpu


def _sort_with_workspace(ids, E):
    L = lib()
    n = ids.numel()
    out = torch.empty_like(ids)
    counts = torch.empty(E, dtype=torch.int32, device=ids.device)
    nbytes = int(L.fx_moe_sort_ws_bytes(max(n, 1), E))
    ws = torch.empty(nbytes // 4, dtype=torch.int32, device=ids.device)
    rc = L.fx_moe_sort(ids.data_ptr(), int(ids.dtype == torch.int64), n, E, out.data_ptr(),
                       int(out.dtype == torch.int64), counts.data_ptr(), None, ws.data_ptr(), nbytes,
                       torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    return out, counts


def _sort_noalloc(ids, E, out, counts, pinned=None):
    rc = lib().fx_moe_sort_noalloc(ids.data_ptr(), int(ids.dtype == torch.int64), ids.numel(), E, out.data_ptr(),
                                   int(out.dtype == torch.int64), counts.data_ptr(),
                                   pinned.data_ptr() if pinned is not None else None,
                                   torch.cuda.current_stream().cuda_stream)
    return rc


def test_noalloc_sort_matches_the_workspace_sort_twice_in_a_row(dev):
    L = lib()
    assert L.fx_moe_sort_noalloc_init() == 0
    g = gen(2024)
    cases = [(131072, 8, 128, torch.int32),     # 1 Mi pairs: 4096 chunks x 128 experts of scratch
             (1000, 2, 8, torch.int64),         # then a much smaller problem on the same array
             (8192, 8, 128, torch.int32),       # the Qwen3-30B-A3B block
             (1, 1, 3, torch.int32), (300, 8, 256, torch.int32)]
    for T, K, E, idt in cases:
        ids = torch.randint(0, E, (T, K), generator=g).to(idt)
        if E >= 8:
            ids[ids == 2] = 5                    # an expert without rows
        d = ids.to(dev)
        want_map, want_counts = _sort_with_workspace(d, E)
        got_map = torch.full_like(d, -7)
        got_counts = torch.full((E,), -7, dtype=torch.int32, device=dev)
        pinned = torch.full((E,), -7, dtype=torch.int32).pin_memory()
        before = torch.cuda.memory_allocated()
        assert _sort_noalloc(d, E, got_map, got_counts, pinned) == 0
        assert torch.cuda.memory_allocated() == before
        torch.cuda.synchronize()
        assert torch.equal(got_map, want_map), (T, K, E)
        assert torch.equal(got_counts, want_counts) and torch.equal(pinned, want_counts.cpu())
        assert int(got_counts.sum()) == T * K
        # and against the definition: a stable argsort by expert
        order = torch.argsort(ids.reshape(-1).long(), stable=True)
        ref = torch.empty(T * K, dtype=torch.int64)
        ref[order] = torch.arange(T * K)
        assert torch.equal(got_map.cpu().reshape(-1).long(), ref)


def test_noalloc_sort_rejects_what_does_not_fit(dev, capfd):
    L = lib()
    words = int(L.fx_moe_sort_noalloc_max_words())
    assert words == 2 * 1024 * 1024 + 1024
    E = 512
    n_fit = (words - 2 * E) // E * 256                     # E * ceil(n / 256) + 2 E == words
    ids = torch.zeros(n_fit + 256, dtype=torch.int32, device=dev)
    out = torch.empty_like(ids)
    counts = torch.empty(E, dtype=torch.int32, device=dev)
    assert _sort_noalloc(ids, E, out, counts) == -1        # one chunk too many
    assert "built-in array" in capfd.readouterr().err
    assert _sort_noalloc(ids[:n_fit], E, out[:n_fit], counts) == 0
    torch.cuda.synchronize()
    assert int(counts[0]) == n_fit and torch.equal(out[:n_fit].cpu(), torch.arange(n_fit, dtype=torch.int32))
    assert _sort_noalloc(ids[:0], E, out[:0], counts) == 0   # empty input: counts all zero
    torch.cuda.synchronize()
    assert not counts.any()
