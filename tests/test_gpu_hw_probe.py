"""The hardware probe on the GPU with short windows: figures are positive, within what the part
can do, and feed a HardwareCost the planner accepts."""
import pytest

from flextrain_amd.hw_probe import probe_hardware
from flextrain_amd.save_level import HardwareCost

pytestmark = pytest.mark.gpu


def test_probe_short_windows(dev):
    r = probe_hardware(device=dev, matmul_n=4096, mem_bw_n=4096, transfer_mib=64, matmul_target_seconds=0.4,
                       mem_bw_target_seconds=0.2, min_matmul_reps_per_half=10, min_mem_bw_reps_per_half=10,
                       n_transfer_reps=3)
    assert isinstance(r.hw_cost, HardwareCost)
    assert r.hw_cost.peak_tflops == r.achieved_tflops_second_half
    assert 50.0 < r.achieved_tflops_second_half < 2600.0 and 50.0 < r.achieved_tflops_first_half < 2600.0
    assert 500.0 < r.mem_bw_gbps < 8100.0
    assert 5.0 < r.hw_cost.pcie_bw_gbps < 70.0
    assert r.matmul_total_seconds >= 0.4 and r.mem_bw_total_seconds >= 0.2
    assert r.transfer_bytes == 64 << 20 and r.matmul_per_call_ms > 0 and r.transfer_per_call_ms > 0
    assert r.hw_cost.flops_to_ms(1e12) > 0 and r.hw_cost.bytes_to_ms(1e9) > 0
