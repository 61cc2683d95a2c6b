"""Save-level planning: from layers and hardware figures to the inputs of the DP solver and from
its answer to the per-(layer, chunk) plan the engine follows.

Host-side mirror of flextrain/core/save_level.py:55-494 (``SaveLevel``, ``SaveLevelPlan``,
``HardwareCost``, ``DPTables``, ``build_dp_tables``, ``plan_from_solution``), same names, fields
and decisions.  A "layer" here is anything with ``layer_id``, ``schema`` (an
``ActivationSchema``) and ``compute_cost(chunk)`` returning ``total_fwd_flops`` and
``avoided_recompute_flops`` per tier; a "chunk" is anything with ``total_q`` tokens.
The solver itself is ``flextrain_amd.transmission_scheduler.TransmissionScheduler``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Mapping, Sequence

import numpy as np


@dataclass(frozen=True, order=True)
class SaveLevel:
    """A tier of the layer's schema (``value >= 0``) or ``-1``: the pair stays in the HBM
    activation ring and has no home slot."""

    value: int

    @staticmethod
    def on_device() -> "SaveLevel":
        return SaveLevel(-1)

    @property
    def is_on_device(self) -> bool:
        return self.value == -1

    @staticmethod
    def all_tiers(schema) -> tuple:
        return tuple(SaveLevel(i) for i in range(schema.max_tier + 1))


@dataclass
class SaveLevelPlan:
    choices: Mapping
    estimated_recompute_time_ms: float
    estimated_fwd_time_ms: float

    def level_for(self, layer_id: int, chunk_id: int) -> SaveLevel:
        return self.choices[(layer_id, chunk_id)]

    @property
    def recompute_fraction(self) -> float:
        if self.estimated_fwd_time_ms <= 0:
            return 0.0
        return self.estimated_recompute_time_ms / self.estimated_fwd_time_ms

    @classmethod
    def all_on_device(cls, layer_ids: Sequence[int], chunk_ids: Sequence[int]) -> "SaveLevelPlan":
        level = SaveLevel.on_device()
        return cls({(l, c): level for l in layer_ids for c in chunk_ids}, 0.0, 0.0)


@dataclass(frozen=True)
class HardwareCost:
    """Measured (sustained) figures that turn FLOPs and bytes into milliseconds."""

    peak_tflops: float
    pcie_bw_gbps: float
    practical_efficiency_factor: float = 1.0

    @property
    def effective_flops_per_ms(self) -> float:
        return self.practical_efficiency_factor * self.peak_tflops * 1e12 / 1e3

    @property
    def pcie_bytes_per_ms(self) -> float:
        return self.pcie_bw_gbps * 1e9 / 1e3

    def flops_to_ms(self, flops: float) -> float:
        rate = self.effective_flops_per_ms
        return flops / rate if rate > 0 else 0.0

    def bytes_to_ms(self, nbytes: float) -> float:
        rate = self.pcie_bytes_per_ms
        return nbytes / rate if rate > 0 else 0.0


@dataclass
class DPTables:
    """Rectangular solver inputs over the T = layers x chunks tasks in forward order: compute
    time per task, and per (task, level) the transfer time, the recompute time saved and the
    home-slot bytes.  Levels a layer does not have carry value -1e18 and duration +1e18."""

    compute_times: np.ndarray
    transfer_durations: np.ndarray
    values: np.ndarray
    home_sizes: np.ndarray
    k_global: int
    indexing: Mapping
    max_tier_per_task: np.ndarray

    @property
    def T(self) -> int:
        return self.compute_times.shape[0]


_NEG_INF = -1e18
_POS_INF = 1e18


def build_dp_tables(layers: Sequence, chunk_metas: Sequence, dims: Mapping[str, int], hw: HardwareCost) -> DPTables:
    """Task t = (layer, chunk) in the order the forward pass visits them (layer-major)."""
    n_tasks = len(layers) * len(chunk_metas)
    k_global = max(layer.schema.max_tier + 1 for layer in layers)
    compute_times = np.zeros(n_tasks, dtype=np.float64)
    transfer = np.full((n_tasks, k_global), _POS_INF, dtype=np.float64)
    values = np.full((n_tasks, k_global), _NEG_INF, dtype=np.float64)
    home = np.zeros((n_tasks, k_global), dtype=np.int64)
    max_tier = np.zeros(n_tasks, dtype=np.int32)
    indexing = {}
    t = 0
    for layer in layers:
        tiers = layer.schema.max_tier + 1
        for chunk_idx, chunk in enumerate(chunk_metas):
            indexing[(layer.layer_id, chunk_idx)] = t
            cost = layer.compute_cost(chunk)
            compute_times[t] = hw.flops_to_ms(cost.total_fwd_flops)
            for level in range(tiers):
                transfer[t, level] = hw.bytes_to_ms(layer.schema.offloaded_bytes_at_level(chunk.total_q, dims, level))
                values[t, level] = hw.flops_to_ms(cost.avoided_recompute_flops[level])
                home[t, level] = layer.schema.home_size_bytes(chunk.total_q, dims, level)
            max_tier[t] = tiers - 1
            t += 1
    return DPTables(compute_times, transfer, values, home, k_global, indexing, max_tier)


def _raise_host_overflow(chosen_bytes, budget, max_total_round_tokens, total_round_tokens) -> None:
    msg = (f"Minimally saving all activations, but still not enough host buffer space "
           f"{chosen_bytes / (1 << 30):.2f}GiB vs. {budget / (1 << 30):.2f}GiB. Reduce max tokens per round")
    if max_total_round_tokens is not None:
        msg += f" below current value of {max_total_round_tokens}"
    if total_round_tokens is not None:
        msg += f" (current round used {total_round_tokens} tokens)"
    raise RuntimeError(msg + ".")


def _demote_to_fit(choices: np.ndarray, sizes: np.ndarray, values: np.ndarray, top_level: int, budget: int,
                   max_total_round_tokens, total_round_tokens) -> None:
    """Lower the levels in ``choices`` (in place) until their home slots fit ``budget`` bytes:
    first every task at the top level one step down, task by task in forward order, then the
    next level, down to level 1; then level 1 -> 0, cheapest lost saving first.  Stops as soon as
    enough bytes are freed (flextrain/core/save_level.py:353-421)."""
    n = choices.shape[0]
    total = int(sizes[np.arange(n), choices].sum())
    if total <= budget:
        return
    floor = int(sizes[:, 0].sum())
    if floor > budget:
        _raise_host_overflow(floor, budget, max_total_round_tokens, total_round_tokens)
    need = total - budget
    freed = 0
    for level in range(top_level, 1, -1):
        if freed >= need:
            break
        for i in np.where(choices == level)[0]:
            freed += int(sizes[i, level] - sizes[i, level - 1])
            choices[i] = level - 1
            if freed >= need:
                break
    if freed < need:
        at_one = np.where(choices == 1)[0]
        for i in at_one[np.argsort(values[at_one, 1])] if at_one.size else ():
            freed += int(sizes[i, 1] - sizes[i, 0])
            choices[i] = 0
            if freed >= need:
                break
    if freed < need:
        _raise_host_overflow(int(sizes[np.arange(n), choices].sum()), budget, max_total_round_tokens, total_round_tokens)
    assert int(sizes[np.arange(n), choices].sum()) <= budget


def plan_from_solution(tables: DPTables, choices_flat, n_gpu_act_slots: int, *, min_required_recompute_time_ms: float,
                       max_optional_recompute_time_avoided_ms: float, host_act_buffer_size: int | None = None,
                       max_total_round_tokens: int | None = None, total_round_tokens: int | None = None) -> SaveLevelPlan:
    """The solver's flat answer (or ``None``: no feasible schedule, everything at tier 0) as a plan.
    Choices above a task's own top tier are clamped; the first ``T - n_gpu_act_slots`` tasks keep
    their (possibly demoted) tiers and need home slots, the last ``n_gpu_act_slots`` stay in the HBM
    ring (level -1) and count as saved at their top tier in the recompute estimate."""
    n_tasks = tables.T
    n_home = max(0, n_tasks - n_gpu_act_slots)
    if choices_flat is None:
        chosen = np.zeros(n_tasks, dtype=np.int32)
    else:
        chosen = np.asarray(choices_flat, dtype=np.int32).copy()
    chosen = np.minimum(chosen, tables.max_tier_per_task.astype(np.int32))

    if host_act_buffer_size is not None and n_home > 0:
        head = chosen[:n_home]           # a view: demotions land in `chosen`
        _demote_to_fit(head, tables.home_sizes[:n_home], tables.values[:n_home],
                       int(tables.max_tier_per_task[:n_home].max(initial=0)), host_act_buffer_size,
                       max_total_round_tokens, total_round_tokens)

    total_fwd = float(tables.compute_times.sum())
    head_saved = float(tables.values[np.arange(n_home), chosen[:n_home]].sum()) if n_home > 0 else 0.0
    if head_saved < -1e15:
        head_saved = 0.0
    tail_saved = (float(tables.values[np.arange(n_home, n_tasks), tables.max_tier_per_task[n_home:n_tasks]].sum())
                  if n_tasks > n_home else 0.0)
    if tail_saved < -1e15:
        tail_saved = 0.0
    recompute = max(0.0, total_fwd - min_required_recompute_time_ms - (head_saved + tail_saved))

    chosen[n_home:] = -1
    choices = {key: SaveLevel(int(chosen[t])) for key, t in tables.indexing.items()}
    return SaveLevelPlan(choices, recompute, total_fwd)


def plan_save_levels(layers: Sequence, chunk_metas: Sequence, dims: Mapping[str, int], hw: HardwareCost,
                     n_gpu_act_slots: int, *, host_act_buffer_size: int | None = None,
                     max_total_round_tokens: int | None = None, force_saved_act_level: int | None = None,
                     solver=None) -> SaveLevelPlan:
    """One round's plan, as the engine derives it (flextrain/engine/active_model.py:874-950): when
    every (layer, chunk) pair fits the HBM ring nothing is offloaded and the solver is skipped;
    otherwise build the tables, run the DP solver, fit the answer to the host buffer, and apply the
    optional forced level to the pairs that do go home (clamped to each layer's top tier)."""
    n_pairs = len(layers) * len(chunk_metas)
    if max(0, n_pairs - n_gpu_act_slots) == 0:
        return SaveLevelPlan.all_on_device([layer.layer_id for layer in layers], list(range(len(chunk_metas))))
    tables = build_dp_tables(layers, chunk_metas, dims, hw)
    max_achievable = float(tables.values[np.arange(tables.T), tables.max_tier_per_task].sum())
    min_required_ms = float(tables.compute_times.sum() - max_achievable)
    if solver is None:
        from .transmission_scheduler import TransmissionScheduler
        solver = TransmissionScheduler()
    _saved, choices = solver.solve(tables.compute_times, tables.transfer_durations, tables.values, n_gpu_act_slots)
    plan = plan_from_solution(tables, choices, n_gpu_act_slots, min_required_recompute_time_ms=min_required_ms,
                              max_optional_recompute_time_avoided_ms=max_achievable,
                              host_act_buffer_size=host_act_buffer_size, max_total_round_tokens=max_total_round_tokens,
                              total_round_tokens=sum(c.total_q for c in chunk_metas))
    if force_saved_act_level is not None:
        by_id = {layer.layer_id: layer for layer in layers}
        forced = {key: (lvl if lvl.is_on_device else SaveLevel(min(int(force_saved_act_level), by_id[key[0]].schema.max_tier)))
                  for key, lvl in plan.choices.items()}
        plan = SaveLevelPlan(forced, plan.estimated_recompute_time_ms, plan.estimated_fwd_time_ms)
    return plan
