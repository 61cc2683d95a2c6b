"""Save-level planning on the CPU: table construction against hand arithmetic, the plan built
from a solver answer (clamping, on-device tail, recompute estimate), host-buffer demotion order,
and an end-to-end plan through the DP solver of the library (host C++ code, no GPU needed)."""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from flextrain_amd.activation_schema import ActivationField, ActivationSchema
from flextrain_amd.save_level import (
    DPTables,
    HardwareCost,
    SaveLevel,
    SaveLevelPlan,
    build_dp_tables,
    plan_from_solution,
    plan_save_levels,
)

bf = torch.bfloat16
DIMS = {"d": 64, "F": 256}


class Layer:
    def __init__(self, layer_id, max_tier):
        self.layer_id = layer_id
        fields = [ActivationField("x_inp", lambda T, m: (T, m["d"]), bf, 0)]
        if max_tier >= 1:
            fields.append(ActivationField("attn", lambda T, m: (T, m["d"]), bf, 1))
        if max_tier >= 2:
            fields.append(ActivationField("x1", lambda T, m: (T, m["F"]), bf, 2))
        self.schema = ActivationSchema(tuple(fields), max_tier=max_tier)

    def compute_cost(self, chunk):
        T = chunk.total_q
        total = 1000 * T
        avoided = (0, 300 * T, 800 * T)[: self.schema.max_tier + 1]
        return SimpleNamespace(total_fwd_flops=total, avoided_recompute_flops=avoided)


def test_hardware_cost_units():
    hw = HardwareCost(peak_tflops=2.0, pcie_bw_gbps=50.0, practical_efficiency_factor=0.5)
    assert hw.effective_flops_per_ms == 1e9 and hw.pcie_bytes_per_ms == 5e7
    assert hw.flops_to_ms(3e9) == 3.0 and hw.bytes_to_ms(1e8) == 2.0
    assert HardwareCost(0.0, 0.0).flops_to_ms(5) == 0.0 and HardwareCost(0.0, 0.0).bytes_to_ms(5) == 0.0
    assert SaveLevel.on_device().is_on_device and SaveLevel(2) > SaveLevel(1)
    assert [s.value for s in SaveLevel.all_tiers(Layer(0, 2).schema)] == [0, 1, 2]


def test_build_tables_heterogeneous_layers():
    layers = [Layer(10, 2), Layer(11, 1)]
    chunks = [SimpleNamespace(total_q=100), SimpleNamespace(total_q=40)]
    hw = HardwareCost(peak_tflops=1e-6, pcie_bw_gbps=1e-3)      # 1e3 flop/ms, 1e3 bytes/ms
    t = build_dp_tables(layers, chunks, DIMS, hw)
    assert t.T == 4 and t.k_global == 3
    assert t.indexing == {(10, 0): 0, (10, 1): 1, (11, 0): 2, (11, 1): 3}
    np.testing.assert_allclose(t.compute_times, [100.0, 40.0, 100.0, 40.0])
    # bytes: x_inp = T*64*2, attn the same, x1 = T*256*2
    np.testing.assert_allclose(t.transfer_durations[0], [12.8, 25.6, 76.8])
    np.testing.assert_allclose(t.values[1], [0.0, 12.0, 32.0])
    assert t.transfer_durations[2, 2] == 1e18 and t.values[3, 2] == -1e18 and t.home_sizes[2, 2] == 0
    assert list(t.max_tier_per_task) == [2, 2, 1, 1]
    assert t.home_sizes[0, 1] == 12800 * 2 and t.home_sizes[1, 0] == 5120      # multiples of 256 already
    assert t.home_sizes[3, 1] == 2 * 5120


def _tables(sizes, values, compute=None, max_tier=None):
    sizes = np.asarray(sizes, dtype=np.int64)
    T, k = sizes.shape
    return DPTables(compute_times=np.asarray(compute if compute is not None else [10.0] * T),
                    transfer_durations=np.zeros((T, k)), values=np.asarray(values, dtype=np.float64),
                    home_sizes=sizes, k_global=k, indexing={(t, 0): t for t in range(T)},
                    max_tier_per_task=np.asarray(max_tier if max_tier is not None else [k - 1] * T, dtype=np.int32))


def test_plan_tail_on_device_clamp_and_estimate():
    t = _tables([[1, 2, 3]] * 4, [[0, 2, 5]] * 4, max_tier=[2, 1, 2, 2])
    plan = plan_from_solution(t, np.array([2, 2, 0, 1]), 1, min_required_recompute_time_ms=4.0,
                              max_optional_recompute_time_avoided_ms=0.0)
    assert [plan.level_for(i, 0).value for i in range(4)] == [2, 1, 0, -1]      # task 1 clamped, task 3 in the ring
    # saved: 5 + 2 + 0 (head) + 5 (tail at its top tier) = 12; forward 40; required 4
    assert plan.estimated_fwd_time_ms == 40.0 and plan.estimated_recompute_time_ms == 24.0
    assert plan.recompute_fraction == 0.6
    none = plan_from_solution(t, None, 1, min_required_recompute_time_ms=0.0, max_optional_recompute_time_avoided_ms=0.0)
    assert [none.level_for(i, 0).value for i in range(4)] == [0, 0, 0, -1]
    assert SaveLevelPlan.all_on_device([1, 2], [0, 1]).level_for(2, 1).is_on_device
    assert SaveLevelPlan({}, 1.0, 0.0).recompute_fraction == 0.0


def test_host_buffer_demotion_order():
    sizes = [[10, 30, 70]] * 5
    values = [[0, 9, 20], [0, 3, 20], [0, 7, 20], [0, 1, 20], [0, 5, 20]]
    t = _tables(sizes, values)
    kw = dict(min_required_recompute_time_ms=0.0, max_optional_recompute_time_avoided_ms=0.0)
    lv = lambda p: [p.level_for(i, 0).value for i in range(5)]
    # all at 2 = 350 bytes; budget 300 -> free 50: tasks 0 and 1 step down (40 each), in forward order
    assert lv(plan_from_solution(t, np.full(5, 2), 0, host_act_buffer_size=300, **kw)) == [1, 1, 2, 2, 2]
    # budget 150 = all at level 1 exactly
    assert lv(plan_from_solution(t, np.full(5, 2), 0, host_act_buffer_size=150, **kw)) == [1, 1, 1, 1, 1]
    # budget 100: 50 more -> level 1 -> 0 for the cheapest savings first: tasks 3 (1), 1 (3), 4 (5)
    assert lv(plan_from_solution(t, np.full(5, 2), 0, host_act_buffer_size=100, **kw)) == [1, 0, 1, 0, 0]
    # the ring tail is not counted against the host buffer
    assert lv(plan_from_solution(t, np.full(5, 2), 2, host_act_buffer_size=210, **kw)) == [2, 2, 2, -1, -1]
    with pytest.raises(RuntimeError, match="Reduce max tokens per round below current value of 4096"):
        plan_from_solution(t, np.full(5, 2), 0, host_act_buffer_size=49, max_total_round_tokens=4096, **kw)
    # fits: untouched
    assert lv(plan_from_solution(t, np.array([2, 0, 1, 0, 2]), 0, host_act_buffer_size=1000, **kw)) == [2, 0, 1, 0, 2]


def test_plan_save_levels_end_to_end_with_the_solver():
    layers = [Layer(i, 2) for i in range(4)]
    chunks = [SimpleNamespace(total_q=512), SimpleNamespace(total_q=256)]
    # everything fits the ring: no solver, all on device
    p = plan_save_levels(layers, chunks, DIMS, HardwareCost(100.0, 50.0), n_gpu_act_slots=8)
    assert all(v.is_on_device for v in p.choices.values())
    # fast link: everything can be saved at the top tier; the last 2 pairs stay in the ring
    fast = plan_save_levels(layers, chunks, DIMS, HardwareCost(peak_tflops=1e-6, pcie_bw_gbps=1.0), n_gpu_act_slots=2)
    vals = [fast.level_for(l, c).value for l in range(4) for c in range(2)]
    assert vals == [2] * 6 + [-1, -1]
    # slow link: transfers do not fit between arrivals, the plan backs off but stays valid
    slow = plan_save_levels(layers, chunks, DIMS, HardwareCost(peak_tflops=1e-6, pcie_bw_gbps=3e-4), n_gpu_act_slots=2)
    sv = [slow.level_for(l, c).value for l in range(4) for c in range(2)]
    assert sv[-2:] == [-1, -1] and all(0 <= v <= 2 for v in sv[:-2]) and sum(sv[:-2]) < 12
    assert slow.estimated_recompute_time_ms > fast.estimated_recompute_time_ms
    forced = plan_save_levels(layers, chunks, DIMS, HardwareCost(1e-6, 1.0), n_gpu_act_slots=2, force_saved_act_level=1)
    assert [forced.level_for(l, c).value for l in range(4) for c in range(2)] == [1] * 6 + [-1, -1]
    small = plan_save_levels(layers, chunks, DIMS, HardwareCost(1e-6, 1.0), n_gpu_act_slots=2,
                             host_act_buffer_size=6 * 512 * 64 * 2)
    assert sum(layers[0].schema.home_size_bytes(chunks[c].total_q, DIMS, small.level_for(l, c).value)
               for l in range(4) for c in range(2) if not small.level_for(l, c).is_on_device) <= 6 * 512 * 64 * 2
