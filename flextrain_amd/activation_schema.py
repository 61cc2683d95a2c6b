"""Tiered activation slots and their host <-> HBM streaming.

Mirror of the reference's activation-slot layer (flextrain/core/activation_schema.py:113-546):
a layer declares its saved tensors once as :class:`ActivationField` s, the
:class:`ActivationSchema` derives sizes and layout, :class:`ActivationSlot` is the typed view over
one flat byte buffer (the pinned host "home" slot sized for the chunk's tokens, or a slot of the
HBM ring sized for the largest chunk), and :func:`send_home` / :func:`fetch_home` move the
offloadable fields of a save level between the two.

Layout rules are the reference's: every field starts on a 256-byte boundary, a slot's size is
rounded up to 256 bytes, fields are packed in declaration order.  Unlike the reference, which
issues one tensor copy per field, a slot is moved by ONE call into the HIP library
(``fx_copy_fields``): contiguous fields as linear DMA copies, fields narrowed along an inner axis
(``softmax_lse`` is ``(heads, tokens)``) as 2-D copies, all enqueued on the current stream.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Callable, Mapping, Sequence

import torch

from ._lib import check, lib, stream_ptr

ShapeFn = Callable[[int, Mapping[str, int]], tuple]

_SLOT_ALIGN_BYTES = 256
_FIELD_ALIGN_BYTES = 256


def _round_up(n: int, align: int) -> int:
    return (n + align - 1) // align * align


def _padded_layout_bytes(fields, num_tokens: int, dims: Mapping[str, int]) -> int:
    offset = 0
    for f in fields:
        offset = _round_up(offset, max(_FIELD_ALIGN_BYTES, f.dtype.itemsize))
        offset += f.byte_size(num_tokens, dims)
    return _round_up(offset, _SLOT_ALIGN_BYTES)


@dataclass(frozen=True)
class ActivationField:
    """One saved tensor: ``shape_fn(num_tokens, dims)`` gives its shape; save level ``L`` keeps the
    fields with ``tier <= L``; ``offload=False`` fields never leave the device; ``persist=False``
    fields are engine scratch without a home slot; ``token_axis`` is the axis that scales with
    the token count (``None``: the block slices the field itself)."""

    name: str
    shape_fn: ShapeFn
    dtype: torch.dtype
    tier: int
    offload: bool = True
    persist: bool = True
    token_axis: int | None = 0

    def shape(self, num_tokens: int, dims: Mapping[str, int]) -> tuple:
        return tuple(self.shape_fn(num_tokens, dims))

    def numel(self, num_tokens: int, dims: Mapping[str, int]) -> int:
        n = 1
        for s in self.shape(num_tokens, dims):
            n *= s
        return n

    def byte_size(self, num_tokens: int, dims: Mapping[str, int]) -> int:
        return self.numel(num_tokens, dims) * self.dtype.itemsize


@dataclass(frozen=True)
class ActivationSchema:
    fields: tuple
    max_tier: int

    def __post_init__(self) -> None:
        names = [f.name for f in self.fields]
        if len(names) != len(set(names)):
            raise ValueError(f"duplicate field names: {sorted({n for n in names if names.count(n) > 1})}")
        for f in self.fields:
            if not (0 <= f.tier <= self.max_tier):
                raise ValueError(f"field {f.name!r} has tier={f.tier}, max_tier={self.max_tier}")

    def fields_at_level(self, level: int) -> tuple:
        return () if level < 0 else tuple(f for f in self.fields if f.tier <= level)

    def has_field(self, name: str) -> bool:
        return any(f.name == name for f in self.fields)

    def _field_tiers_cache(self) -> dict:
        return {f.name: f.tier for f in self.fields}

    def persistent_fields_at_level(self, level: int) -> tuple:
        return tuple(f for f in self.fields_at_level(level) if f.persist)

    def offloadable_fields_at_level(self, level: int) -> tuple:
        return tuple(f for f in self.persistent_fields_at_level(level) if f.offload)

    def device_fields(self) -> tuple:
        return self.fields

    def home_size_bytes(self, num_tokens: int, dims: Mapping[str, int], level: int) -> int:
        """Bytes of the pinned home slot of one (chunk, layer) at a save level."""
        return _padded_layout_bytes(self.persistent_fields_at_level(level), num_tokens, dims)

    def device_size_bytes(self, num_tokens: int, dims: Mapping[str, int]) -> int:
        """Bytes of a slot of the HBM activation ring: every field of every tier."""
        return _padded_layout_bytes(self.fields, num_tokens, dims)

    def offloaded_bytes_at_level(self, num_tokens: int, dims: Mapping[str, int], level: int) -> int:
        """Bytes that cross the host link at this save level (what the save-level solver prices)."""
        return sum(f.byte_size(num_tokens, dims) for f in self.offloadable_fields_at_level(level))


class ActivationSlot:
    """Typed view over the tensors of one (chunk, layer) pair: ``slot.x_inp``, ``slot.has(name)``,
    ``slot.aux`` for hand-offs between a block's forward / backward helpers."""

    __slots__ = ("schema", "level", "_tensors", "aux")

    def __init__(self, schema: ActivationSchema, level: int, tensors: Mapping[str, torch.Tensor]) -> None:
        self.schema = schema
        self.level = level
        self._tensors = dict(tensors)
        self.aux = {}

    def __getattr__(self, name: str) -> torch.Tensor:
        try:
            return self._tensors[name]
        except KeyError:
            raise AttributeError(f"activation field {name!r} not present at level={self.level} "
                                 f"(available: {sorted(self._tensors)})") from None

    def has(self, name: str) -> bool:
        """Whether the field is VALID at this slot's save level: a declared field counts only when
        its tier is within the level, even if a (stale) view of it exists in the slot."""
        tier = self.schema._field_tiers_cache().get(name)
        if tier is None:
            return name in self._tensors
        return tier <= self.level

    def set(self, name: str, tensor: torch.Tensor) -> None:
        self._tensors[name] = tensor

    def items(self):
        return self._tensors.items()

    def __repr__(self) -> str:
        return f"ActivationSlot(level={self.level}, fields={sorted(self._tensors)})"

    @classmethod
    def from_buffer(cls, schema: ActivationSchema, level: int, num_tokens: int, dims: Mapping[str, int],
                    buffer: torch.Tensor, *, include_nonpersistent: bool = False):
        """Slice a 1-D uint8 ``buffer`` into the fields of ``level``; returns the slot and the bytes
        consumed (equal to ``home_size_bytes`` / ``device_size_bytes``)."""
        if buffer.dtype is not torch.uint8 or buffer.dim() != 1:
            raise TypeError("buffer must be a 1-D uint8 tensor")
        fields = schema.fields_at_level(level) if include_nonpersistent else schema.persistent_fields_at_level(level)
        tensors = {}
        offset = 0
        for f in fields:
            shape = f.shape(num_tokens, dims)
            nbytes = f.byte_size(num_tokens, dims)
            offset = _round_up(offset, max(_FIELD_ALIGN_BYTES, f.dtype.itemsize))
            if offset + nbytes > buffer.numel():
                raise ValueError(f"buffer too small: field {f.name!r} needs {nbytes}B at offset {offset}, "
                                 f"buffer has {buffer.numel()}B")
            tensors[f.name] = buffer[offset:offset + nbytes].view(f.dtype).reshape(shape)
            offset += nbytes
        return cls(schema, level, tensors), _round_up(offset, _SLOT_ALIGN_BYTES)

    def view_for(self, num_tokens: int, dims: Mapping[str, int]) -> "ActivationSlot":
        """Every tensor narrowed to the first ``num_tokens`` along its token axis."""
        by_name = {f.name: f for f in self.schema.fields}
        narrowed = {}
        for name, tensor in self._tensors.items():
            axis = by_name[name].token_axis if name in by_name else None
            if axis is None or tensor.shape[axis] == num_tokens:
                narrowed[name] = tensor
            else:
                narrowed[name] = tensor.narrow(axis, 0, num_tokens)
        return ActivationSlot(self.schema, self.level, narrowed)


def _match_to(src: torch.Tensor, dst: torch.Tensor) -> torch.Tensor:
    """View of ``src`` cut down to ``dst``'s shape (the HBM ring is sized for the largest chunk,
    the home slot for the chunk's own tokens)."""
    if src.shape == dst.shape:
        return src
    out = src
    for axis, (s, d) in enumerate(zip(src.shape, dst.shape)):
        if s != d:
            if s < d:
                raise ValueError(f"send_home/fetch_home: source shape {tuple(src.shape)} smaller than dest "
                                 f"{tuple(dst.shape)} at axis {axis}")
            out = out.narrow(axis, 0, d)
    return out


def _as_rows(t: torch.Tensor):
    """``(rows, row_bytes, pitch_bytes)`` of a tensor that is ``rows`` equal contiguous pieces a
    constant pitch apart (a contiguous tensor is one piece), or ``None`` when it has no such form.
    A view narrowed along one axis of a contiguous tensor always has it."""
    es = t.element_size()
    if t.numel() == 0:
        return 0, 0, 0
    if t.is_contiguous():
        return 1, t.numel() * es, t.numel() * es
    for k in range(1, t.dim()):            # dims [k:] form the piece, dims [:k] count the pieces
        inner_numel, expect, ok = 1, 1, True
        for d in range(t.dim() - 1, k - 1, -1):
            if t.shape[d] != 1 and t.stride(d) != expect:
                ok = False
                break
            expect *= t.shape[d]
            inner_numel *= t.shape[d]
        if not ok:
            continue
        pitch, rows, expect = t.stride(k - 1), 1, t.stride(k - 1)
        for d in range(k - 1, -1, -1):
            if t.shape[d] != 1 and t.stride(d) != expect:
                ok = False
                break
            expect *= t.shape[d]
            rows *= t.shape[d]
        if ok and pitch >= inner_numel:
            return rows, inner_numel * es, pitch * es
    return None


def _copy_desc(dst: torch.Tensor, src: torch.Tensor):
    """``(rows, row_bytes, dst_pitch, src_pitch)`` for one linear or 2-D copy, or ``None``."""
    rd, rs = _as_rows(dst), _as_rows(src)
    if rd is None or rs is None:
        return None
    if rd[0] == 1 and rs[0] == 1:
        return 1, rd[1], rd[1], rs[1]
    if rd[0] == 1:                          # contiguous destination, pitched source
        return rs[0], rs[1], rs[1], rs[2]
    if rs[0] == 1:                          # pitched destination, contiguous source
        return rd[0], rd[1], rd[2], rd[1]
    if rd[:2] == rs[:2]:                    # both pitched, same pieces
        return rd[0], rd[1], rd[2], rs[2]
    return None


_DIRECTION = {(False, True): 0, (True, False): 1, (True, True): 2}    # (dst on device, src on device)


def copy_fields(pairs: Sequence[tuple], *, non_blocking: bool = True) -> None:
    """Copy ``src -> dst`` for every ``(dst, src)`` pair with one library call per direction, on the
    current stream.  Host tensors must be pinned for the copies to overlap with compute."""
    by_dir = {}
    strided = []
    for dst, src in pairs:
        if dst.shape != src.shape or dst.dtype != src.dtype:
            raise ValueError(f"copy_fields: {tuple(src.shape)} {src.dtype} -> {tuple(dst.shape)} {dst.dtype}")
        if dst.numel() == 0:
            continue
        direction = _DIRECTION.get((dst.is_cuda, src.is_cuda))
        desc = _copy_desc(dst, src) if direction is not None else None
        if desc is None:
            strided.append((dst, src))
            continue
        device = dst.device if dst.is_cuda else src.device
        by_dir.setdefault((direction, device), []).append((dst.data_ptr(), src.data_ptr()) + desc)
    for (direction, device), items in by_dir.items():
        n = len(items)
        P, I = ctypes.c_void_p * n, ctypes.c_int64 * n
        cols = list(zip(*items))
        rc = lib().fx_copy_fields(n, P(*cols[0]), P(*cols[1]), I(*cols[2]), I(*cols[3]), I(*cols[4]), I(*cols[5]),
                                  direction, stream_ptr(device))
        check(rc, "fx_copy_fields")
    for dst, src in strided:               # no single 2-D form (or host to host): the framework's strided copy
        dst.copy_(src, non_blocking=non_blocking)
    if not non_blocking:
        torch.cuda.current_stream().synchronize()


def send_home(home_slot: ActivationSlot, computed_slot: ActivationSlot, level: int, *, non_blocking: bool = True) -> None:
    """Every offloadable field of ``level`` from the device slot into the pinned home slot."""
    if home_slot.schema is not computed_slot.schema:
        raise ValueError("home and computed slots must share a schema")
    pairs = []
    for f in home_slot.schema.offloadable_fields_at_level(level):
        dst = home_slot._tensors[f.name]
        pairs.append((dst, _match_to(computed_slot._tensors[f.name], dst)))
    copy_fields(pairs, non_blocking=non_blocking)


def fetch_home(dest_slot: ActivationSlot, home_slot: ActivationSlot, level: int, *, non_blocking: bool = True) -> None:
    """Every offloadable field of ``level`` from the pinned home slot back into the device slot."""
    if dest_slot.schema is not home_slot.schema:
        raise ValueError("dest and home slots must share a schema")
    pairs = []
    for f in dest_slot.schema.offloadable_fields_at_level(level):
        src = home_slot._tensors[f.name]
        pairs.append((_match_to(dest_slot._tensors[f.name], src), src))
    copy_fields(pairs, non_blocking=non_blocking)


def concat_fields(blocks: Sequence[Sequence[ActivationField]]) -> tuple:
    """Per-block field tuples joined into the flat sequence a schema expects; duplicate names raise."""
    out = []
    for block in blocks:
        out.extend(block)
    names = [f.name for f in out]
    if len(names) != len(set(names)):
        raise ValueError(f"duplicate field names across blocks: {sorted({n for n in names if names.count(n) > 1})}")
    return tuple(out)


class ActivationStreamer:
    """The engine's two activation transfers with their stream and event protocol
    (flextrain/engine/active_model.py:1184-1199 offload after a forward step, :2036-2098 prefetch
    before a backward step), over a ``StreamBundle`` and an ``EventBook``."""

    def __init__(self, streams, events) -> None:
        self.streams = streams
        self.events = events

    def offload(self, key, ring_slot: int, home_slot: ActivationSlot, computed_slot: ActivationSlot, level: int) -> None:
        """Send the slot home on the outbound stream once compute has produced it.  Records
        ``act_slot_ready[ring_slot]`` (the ring slot may be overwritten) and
        ``home_act_slot_available[key]`` (the home copy is complete) on that stream."""
        self.streams.outbound.wait_stream(self.streams.compute)
        with torch.cuda.stream(self.streams.outbound):
            send_home(home_slot, computed_slot, level)
        self.events.act_slot_ready.record_on(ring_slot, self.streams.outbound)
        self.events.home_act_slot_available.record_on(key, self.streams.outbound)

    def prefetch(self, key, full_dev_slot: ActivationSlot, home_slot: ActivationSlot) -> ActivationSlot:
        """Bring a home slot back into a ring slot on the inbound stream.  The returned slot keeps
        every view of the ring slot but carries the SAVED level, so ``has()`` is false for the
        higher-tier fields that still hold another layer's data and must be recomputed."""
        self.streams.inbound.wait_stream(self.streams.compute)
        avail = self.events.home_act_slot_available.get(key)
        if avail is not None:
            self.streams.inbound.wait_event(avail)
        schema, level = home_slot.schema, home_slot.level
        narrowed = ActivationSlot(schema, level, {f.name: full_dev_slot._tensors[f.name]
                                                  for f in schema.persistent_fields_at_level(level) if f.offload})
        with torch.cuda.stream(self.streams.inbound):
            fetch_home(narrowed, home_slot, level)
        dev_slot = ActivationSlot(schema, level, full_dev_slot._tensors)
        self.events.dev_act_slot_mapping[key] = dev_slot
        self.events.inbound_act_slot_ready.record_on(key, self.streams.inbound)
        return dev_slot
