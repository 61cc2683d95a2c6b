"""Per-layer parameter / gradient / optimizer-state rings between pinned host memory and
HBM, and the streamed optimizer step over them.

The accessor names and meanings are those of the reference's ``BufferManager``
(flextrain/engine/buffers.py:981-1034 ``gpu_param_slot`` / ``gpu_grad_slot``; :1088-1164
``fetch_layer_params`` / ``fetch_layer_grads`` / ``offload_layer_grads`` /
``offload_layer_params``; :1170-1297 ``swap_to_optimizer_state`` / ``gpu_opt_slot`` /
``fetch_layer_opt`` / ``offload_layer_opt`` / ``restore_activation_ring``) and
:func:`ring_optimizer_step` is the per-layer pipeline of ``ActiveModel.step``
(flextrain/engine/active_model.py:486-655).  The layout underneath is this package's:

* Each layer's host copy of a role (master params, grads, Adam m, Adam v) is ONE pinned
  allocation; tensors are views at element offsets that are multiples of 128 elements,
  trainable tensors first, frozen ones after them.  A device ring slot has the same
  packing, so fetching or offloading a layer's role is one contiguous DMA of the
  trainable region (the reference issues one ``copy_`` per tensor), and because the
  ELEMENT offsets are the same in every role, the optimizer step of a whole layer is one
  AdamW launch over the flat trainable region instead of one per tensor (padding
  elements are zero in all four roles and stay zero under the update).
* A ring slot holds the host's bytes: there is no cast on the link.  (Rounding master
  weights to the compute dtype belongs in the optimizer kernel: its bf16 copy-out.)
* Every copy is enqueued on an explicitly chosen non-default stream and its completion
  is filed in the ``EventBook``; nothing here touches the null stream
  (flextrain/engine/active_model.py:579-583 records why that matters).
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Sequence

import torch

from ._lib import check, lib
from .host_memory import LocalPinnedHostBackend
from .ops.adamw import flextrain_adamw_step
from .optim import state_key
from .streams import EventBook, StreamBundle

_ALIGN_ELEMS = 128          # 256 bytes for 2-byte elements, 512 for 4-byte ones


@dataclass(frozen=True)
class RingTensor:
    """One parameter tensor of a layer: what the rings need to know of a ``TensorSpec``
    (flextrain/core/layer.py: name, concrete shape, frozen flag)."""
    name: str
    shape: tuple
    frozen: bool = False

    def numel(self) -> int:
        return _numel(self.shape)


@dataclass(frozen=True)
class RingParamSpec:
    """All parameter tensors one layer owns, in spec order."""
    tensors: tuple

    def __post_init__(self):
        names = [t.name for t in self.tensors]
        if len(names) != len(set(names)):
            raise ValueError(f"duplicate parameter names in {names}")


def _up(n: int, a: int = _ALIGN_ELEMS) -> int:
    return (n + a - 1) // a * a


def _numel(shape) -> int:
    n = 1
    for d in shape:
        n *= int(d)
    return n


class _Packing:
    """Element offsets of a layer's tensors inside a slot: the trainable region, and the
    frozen region (offsets relative to that region's base)."""

    def __init__(self, spec) -> None:
        self.trainable: dict[str, tuple[int, tuple]] = {}
        self.frozen: dict[str, tuple[int, tuple]] = {}
        cur_t = cur_f = 0
        for t in spec.tensors:
            shape = tuple(int(d) for d in t.shape)
            if t.frozen:
                self.frozen[t.name] = (cur_f, shape)
                cur_f = _up(cur_f + _numel(shape))
            else:
                self.trainable[t.name] = (cur_t, shape)
                cur_t = _up(cur_t + _numel(shape))
        self.train_elems, self.frozen_elems = cur_t, cur_f


def _copy_region(dst: torch.Tensor, src: torch.Tensor, nbytes: int, direction: int, stream: torch.cuda.Stream) -> None:
    """One contiguous asynchronous copy of ``nbytes`` bytes on ``stream`` (0: device to host, 1: host to device)."""
    if nbytes == 0:
        return
    d, s = (ctypes.c_void_p * 1)(dst.data_ptr()), (ctypes.c_void_p * 1)(src.data_ptr())
    one, nb = (ctypes.c_int64 * 1)(1), (ctypes.c_int64 * 1)(nbytes)
    check(lib().fx_copy_fields(1, d, s, one, nb, nb, nb, direction, stream.cuda_stream), "fx_copy_fields")


class LayerRingBuffers:
    """Host tables of every layer's parameters, gradients and optimizer state, and the
    device rings they rotate through.

    ``layer_specs[i]`` describes layer ``i`` (objects with ``.tensors``, each tensor with
    ``.name``, ``.shape``, ``.frozen``); layers may differ in shape.  ``n_param_slots`` /
    ``n_grad_slots`` size the two device rings (the reference's ``n_gpu_layers`` /
    ``n_gpu_grads``); the optimizer-state ring is carved out of ``gpu_act_ring`` by
    :meth:`swap_to_optimizer_state`, as the reference re-uses its activation ring for the step.
    """

    def __init__(self, layer_specs: Sequence, *, device, n_param_slots: int, n_grad_slots: int, act_ring_bytes: int,
                 param_dtype=torch.float32, grad_dtype=torch.bfloat16, opt_dtype=torch.float32,
                 opt_state_names=("o_adam_m", "o_adam_v"), host_backend=None) -> None:
        if n_param_slots < 1 or n_grad_slots < 1:
            raise ValueError("rings need at least one slot each")
        self.device = torch.device(device)
        self.layer_param_specs = list(layer_specs)
        self.param_dtype, self.grad_dtype, self.opt_dtype = param_dtype, grad_dtype, opt_dtype
        self.opt_state_names = tuple(opt_state_names)
        self._host = host_backend or LocalPinnedHostBackend()
        self._pack = [_Packing(s) for s in self.layer_param_specs]
        self._max_train = max(p.train_elems for p in self._pack)
        self._max_frozen = max(p.frozen_elems for p in self._pack)
        psz, gsz = torch.empty((), dtype=param_dtype).element_size(), torch.empty((), dtype=grad_dtype).element_size()
        self._param_slot_elems = self._max_train + self._max_frozen
        self.gpu_param_ring = torch.zeros(n_param_slots * self._param_slot_elems, dtype=param_dtype, device=self.device)
        self.gpu_grad_ring = torch.zeros(n_grad_slots * self._max_train, dtype=grad_dtype, device=self.device)
        self.gpu_act_ring = torch.zeros(int(act_ring_bytes), dtype=torch.uint8, device=self.device)
        self.n_param_slots, self.n_grad_slots = n_param_slots, n_grad_slots
        self._psz, self._gsz = psz, gsz
        self._osz = torch.empty((), dtype=opt_dtype).element_size()
        # host tables: one pinned allocation per (layer, role); name -> view dicts over them
        self._host_param_flat, self._host_grad_flat, self._host_opt_flat = [], [], []
        self.host_params, self.host_grads, self.host_opt = [], [], []
        for spec, pk in zip(self.layer_param_specs, self._pack):
            pf = self._host.allocate_tensor((pk.train_elems + pk.frozen_elems,), param_dtype)
            gf = self._host.allocate_tensor((pk.train_elems,), grad_dtype)
            of = [self._host.allocate_tensor((pk.train_elems,), opt_dtype) for _ in self.opt_state_names]
            self._host_param_flat.append(pf)
            self._host_grad_flat.append(gf)
            self._host_opt_flat.append(of)
            self.host_params.append(self._views(pk, pf, 0, pk.train_elems, include_frozen=True, prefix=None))
            self.host_grads.append(self._views(pk, gf, 0, 0, include_frozen=False, prefix="g_"))
            opt = {}
            for sname, flat in zip(self.opt_state_names, of):
                opt.update(self._views(pk, flat, 0, 0, include_frozen=False, prefix=sname))
            self.host_opt.append(opt)
        self._in_opt_mode = False
        self._n_opt_slots = 0

    # ------------------------------------------------------------------ views
    @staticmethod
    def _key(name: str, prefix) -> str:
        if prefix is None:
            return name
        if prefix == "g_":
            return "g_" + (name[2:] if name.startswith("w_") else name)
        return state_key(prefix, name)

    def _views(self, pk: _Packing, flat: torch.Tensor, base: int, frozen_base: int, *, include_frozen: bool, prefix):
        out = {}
        for name, (off, shape) in pk.trainable.items():
            out[self._key(name, prefix)] = flat[base + off: base + off + _numel(shape)].view(shape)
        if include_frozen:
            for name, (off, shape) in pk.frozen.items():
                out[self._key(name, prefix)] = flat[frozen_base + off: frozen_base + off + _numel(shape)].view(shape)
        return out

    def _layer_of(self, layer_spec) -> int:
        for i, s in enumerate(self.layer_param_specs):
            if s is layer_spec:
                return i
        for i, s in enumerate(self.layer_param_specs):
            if s == layer_spec:
                return i
        raise KeyError("layer_spec is not one of this manager's layers")

    def gpu_param_slot(self, slot_idx: int, layer_spec) -> dict:
        """name -> view of ring slot ``slot_idx`` laid out for ``layer_spec``: trainable tensors
        in ``[0, max_train)``, frozen ones from a base that is the same for every layer, so
        writing one layer's trainable region never touches another layer's frozen bytes."""
        if not 0 <= slot_idx < self.n_param_slots:
            raise IndexError(f"param slot {slot_idx} out of range (ring has {self.n_param_slots})")
        pk = self._pack[self._layer_of(layer_spec)]
        base = slot_idx * self._param_slot_elems
        return self._views(pk, self.gpu_param_ring, base, base + self._max_train, include_frozen=True, prefix=None)

    def gpu_grad_slot(self, slot_idx: int, layer_spec) -> dict:
        if not 0 <= slot_idx < self.n_grad_slots:
            raise IndexError(f"grad slot {slot_idx} out of range (ring has {self.n_grad_slots})")
        pk = self._pack[self._layer_of(layer_spec)]
        return self._views(pk, self.gpu_grad_ring, slot_idx * self._max_train, 0, include_frozen=False, prefix="g_")

    # ------------------------------------------------------- optimizer-state ring
    def swap_to_optimizer_state(self, n_gpu_opt_layers: int) -> list:
        """Carve ``n_gpu_opt_layers`` optimizer-state slots out of the activation ring
        (free once forward/backward is over).  Until :meth:`restore_activation_ring` the
        ring must not be used for activations."""
        per_slot = len(self.opt_state_names) * self._max_train * self._osz
        if n_gpu_opt_layers < 1:
            raise ValueError("need at least one optimizer-state slot")
        if n_gpu_opt_layers * per_slot > self.gpu_act_ring.numel():
            raise RuntimeError(f"opt-state ring ({n_gpu_opt_layers} * {per_slot}) exceeds gpu_act_buffer "
                               f"({self.gpu_act_ring.numel()})")
        self._n_opt_slots = n_gpu_opt_layers
        self._opt_slot_bytes = per_slot
        self._in_opt_mode = True
        return []

    def restore_activation_ring(self) -> None:
        self._in_opt_mode = False
        self._n_opt_slots = 0

    def _opt_flat(self, slot_idx: int, which: int) -> torch.Tensor:
        if not self._in_opt_mode:
            raise RuntimeError("gpu_opt_slot called outside swap_to_optimizer_state() window")
        if not 0 <= slot_idx < self._n_opt_slots:
            raise IndexError(f"opt slot {slot_idx} out of range (ring has {self._n_opt_slots})")
        a = slot_idx * self._opt_slot_bytes + which * self._max_train * self._osz
        return self.gpu_act_ring[a: a + self._max_train * self._osz].view(self.opt_dtype)

    def gpu_opt_slot(self, slot_idx: int, layer_id: int) -> dict:
        """``{"o_adam_m_q": ..., "o_adam_v_q": ...}`` views of optimizer-state slot ``slot_idx``
        laid out for layer ``layer_id``."""
        pk = self._pack[layer_id]
        out = {}
        for which, sname in enumerate(self.opt_state_names):
            out.update(self._views(pk, self._opt_flat(slot_idx, which), 0, 0, include_frozen=False, prefix=sname))
        return out

    def flat_trainable(self, layer_id: int, param_slot: int, grad_slot: int, opt_slot: int):
        """The trainable region of a layer as flat tensors ``(p, g, [state...])`` with equal
        element counts and matching element offsets: what a whole-layer optimizer launch takes."""
        n = self._pack[layer_id].train_elems
        pb = param_slot * self._param_slot_elems
        gb = grad_slot * self._max_train
        states = [self._opt_flat(opt_slot, w)[:n] for w in range(len(self.opt_state_names))]
        return self.gpu_param_ring[pb: pb + n], self.gpu_grad_ring[gb: gb + n], states

    # ------------------------------------------------------------ fetch / offload
    @staticmethod
    def _stream(stream):
        s = stream if stream is not None else torch.cuda.current_stream()
        if s.cuda_stream == 0:
            raise RuntimeError("ring copies must be issued on an explicit non-default stream "
                               "(pass stream=, or call inside `with torch.cuda.stream(s)`)")
        return s

    def fetch_layer_params(self, layer_id: int, slot_idx: int, *, non_blocking: bool = True, skip_frozen: bool = False,
                           stream=None) -> None:
        """Host master parameters of ``layer_id`` -> param ring slot ``slot_idx``.
        ``skip_frozen=True`` moves the trainable region only (the optimizer step never
        reads frozen tensors and their device copies stay valid)."""
        s = self._stream(stream)
        pk, host = self._pack[layer_id], self._host_param_flat[layer_id]
        base = slot_idx * self._param_slot_elems
        _copy_region(self.gpu_param_ring[base:], host, pk.train_elems * self._psz, 1, s)
        if not skip_frozen and pk.frozen_elems:
            _copy_region(self.gpu_param_ring[base + self._max_train:], host[pk.train_elems:], pk.frozen_elems * self._psz,
                         1, s)
        if not non_blocking:
            s.synchronize()

    def offload_layer_params(self, layer_id: int, slot_idx: int, *, non_blocking: bool = True, stream=None) -> None:
        """Param ring slot -> host master copy; frozen tensors never change and are skipped."""
        s = self._stream(stream)
        pk = self._pack[layer_id]
        base = slot_idx * self._param_slot_elems
        _copy_region(self._host_param_flat[layer_id], self.gpu_param_ring[base:], pk.train_elems * self._psz, 0, s)
        if not non_blocking:
            s.synchronize()

    def fetch_layer_grads(self, layer_id: int, slot_idx: int, *, non_blocking: bool = True, stream=None) -> None:
        s = self._stream(stream)
        pk = self._pack[layer_id]
        _copy_region(self.gpu_grad_ring[slot_idx * self._max_train:], self._host_grad_flat[layer_id],
                     pk.train_elems * self._gsz, 1, s)
        if not non_blocking:
            s.synchronize()

    def offload_layer_grads(self, layer_id: int, slot_idx: int, *, non_blocking: bool = True, stream=None) -> None:
        s = self._stream(stream)
        pk = self._pack[layer_id]
        _copy_region(self._host_grad_flat[layer_id], self.gpu_grad_ring[slot_idx * self._max_train:],
                     pk.train_elems * self._gsz, 0, s)
        if not non_blocking:
            s.synchronize()

    def fetch_layer_opt(self, layer_id: int, slot_idx: int, *, non_blocking: bool = True, stream=None) -> None:
        s = self._stream(stream)
        pk = self._pack[layer_id]
        for which, flat in enumerate(self._host_opt_flat[layer_id]):
            _copy_region(self._opt_flat(slot_idx, which), flat, pk.train_elems * self._osz, 1, s)
        if not non_blocking:
            s.synchronize()

    def offload_layer_opt(self, layer_id: int, slot_idx: int, *, non_blocking: bool = True, stream=None) -> None:
        s = self._stream(stream)
        pk = self._pack[layer_id]
        for which, flat in enumerate(self._host_opt_flat[layer_id]):
            _copy_region(flat, self._opt_flat(slot_idx, which), pk.train_elems * self._osz, 0, s)
        if not non_blocking:
            s.synchronize()

    def release(self) -> None:
        """Free the pinned host tables (the views handed out become invalid)."""
        for t in self._host_param_flat + self._host_grad_flat + [f for o in self._host_opt_flat for f in o]:
            self._host.release(t)
        self._host_param_flat, self._host_grad_flat, self._host_opt_flat = [], [], []
        self.host_params, self.host_grads, self.host_opt = [], [], []


def ring_optimizer_step(buffers: LayerRingBuffers, streams: StreamBundle, events: EventBook, *, n_gpu_opt_layers: int,
                        step_num: int, lr=1e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.001,
                        optimizer=None, per_tensor: bool = False, synchronize_every_op: bool = False) -> int:
    """The streamed optimizer step over all layers (flextrain/engine/active_model.py:486-655,
    steps 2-5): the first ``N`` layers of every role are prefetched on ``inbound``; then per
    layer ``compute`` waits for its three fetches and updates it, ``outbound`` writes parameters
    and optimizer state back, and ``inbound`` refills the freed slots with the layers ``N``
    positions ahead.  Slot reuse is ordered by events: a refill waits for the offload that
    reads the slot, an offload waits for the kernel that wrote it.

    The update is one AdamW launch over the layer's flat trainable region; ``per_tensor=True``
    (or an ``optimizer`` object with ``step(param_spec, weights, grads, state, step_num=)``,
    the reference's interface) updates tensor by tensor instead.  Returns 0, or the
    optimizer's first non-zero status (the rings are restored either way).
    ``synchronize_every_op=True`` drains all streams after every enqueue: the synchronous
    schedule the pipelined one must equal bit for bit."""
    L = len(buffers.layer_param_specs)
    N_P, N_G, N_O = buffers.n_param_slots, buffers.n_grad_slots, n_gpu_opt_layers
    if len(buffers.opt_state_names) != 2 and optimizer is None:
        raise ValueError("the built-in AdamW step needs exactly two state tensors (m, v)")
    buffers.swap_to_optimizer_state(N_O)
    for m in (events.weight_inbound, events.grad_weight_inbound, events.opt_inbound):
        m.clear()

    def settle():
        if synchronize_every_op:
            streams.synchronize_all()

    inb, comp, outb = streams.inbound, streams.compute, streams.outbound
    # The first fetches overwrite the parameter and gradient rings and the activation ring that now
    # serves as optimizer state, and read host gradients the backward pass offloaded: they must come
    # after everything already enqueued on the compute stream (last backward kernels) and on the
    # outbound stream (gradient offloads).  Device-side order only; the host does not wait.
    for producer in (comp, outb):
        fence = torch.cuda.Event()
        fence.record(producer)
        inb.wait_event(fence)
    for i in range(min(N_P, L)):
        buffers.fetch_layer_params(i, i, skip_frozen=True, stream=inb)
        events.weight_inbound.record_on(i, inb)
    for i in range(min(N_G, L)):
        buffers.fetch_layer_grads(i, i, stream=inb)
        events.grad_weight_inbound.record_on(i, inb)
    for i in range(min(N_O, L)):
        buffers.fetch_layer_opt(i, i, stream=inb)
        events.opt_inbound.record_on(i, inb)
    settle()

    cur_w = cur_g = cur_o = 0
    ret = 0
    for lid in range(L):
        for m in (events.weight_inbound, events.grad_weight_inbound, events.opt_inbound):
            m.wait_on(lid, comp)
        spec = buffers.layer_param_specs[lid]
        with torch.cuda.stream(comp):
            if optimizer is not None:
                ret = optimizer.step(spec, buffers.gpu_param_slot(cur_w, spec), buffers.gpu_grad_slot(cur_g, spec),
                                     buffers.gpu_opt_slot(cur_o, lid), step_num=step_num)
            elif per_tensor:
                w, g, o = (buffers.gpu_param_slot(cur_w, spec), buffers.gpu_grad_slot(cur_g, spec),
                           buffers.gpu_opt_slot(cur_o, lid))
                for t in spec.tensors:
                    if t.frozen:
                        continue
                    gk = "g_" + (t.name[2:] if t.name.startswith("w_") else t.name)
                    ret = flextrain_adamw_step(w[t.name].view(-1), g[gk].view(-1),
                                               o[state_key(buffers.opt_state_names[0], t.name)].view(-1),
                                               o[state_key(buffers.opt_state_names[1], t.name)].view(-1), lr=lr,
                                               beta1=beta1, beta2=beta2, eps=eps, weight_decay=weight_decay,
                                               step=step_num)
                    if ret:
                        break
            else:
                p, g, (m_, v_) = buffers.flat_trainable(lid, cur_w, cur_g, cur_o)
                ret = flextrain_adamw_step(p, g, m_, v_, lr=lr, beta1=beta1, beta2=beta2, eps=eps,
                                           weight_decay=weight_decay, step=step_num)
        if ret:
            break
        updated = comp.record_event()
        settle()
        outb.wait_event(updated)
        buffers.offload_layer_params(lid, cur_w, stream=outb)
        buffers.offload_layer_opt(lid, cur_o, stream=outb)
        written_back = outb.record_event()
        settle()
        # refills: the param and opt slots are read by the offload just enqueued, the grad slot by the kernel
        nxt = lid + N_P
        if nxt < L:
            inb.wait_event(written_back)
            buffers.fetch_layer_params(nxt, cur_w, skip_frozen=True, stream=inb)
            events.weight_inbound.record_on(nxt, inb)
        events.weight_inbound.mark_consumed(lid)
        nxt = lid + N_G
        if nxt < L:
            inb.wait_event(updated)
            buffers.fetch_layer_grads(nxt, cur_g, stream=inb)
            events.grad_weight_inbound.record_on(nxt, inb)
        events.grad_weight_inbound.mark_consumed(lid)
        nxt = lid + N_O
        if nxt < L:
            inb.wait_event(written_back)
            buffers.fetch_layer_opt(nxt, cur_o, stream=inb)
            events.opt_inbound.record_on(nxt, inb)
        events.opt_inbound.mark_consumed(lid)
        settle()
        cur_w, cur_g, cur_o = (cur_w + 1) % N_P, (cur_g + 1) % N_G, (cur_o + 1) % N_O

    streams.synchronize_all()
    buffers.restore_activation_ring()
    return ret


__all__ = ["RingTensor", "RingParamSpec", "LayerRingBuffers", "ring_optimizer_step"]
