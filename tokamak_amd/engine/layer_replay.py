"""Layers of one kind launch the same kernels in a step: record one, replay the others.

A step that is not replayed from a HIP graph (prompt portions, more requests than the
recorded shapes take) pays for every kernel launch in Python: checks of shapes and dtypes,
the choice of a kernel, allocations.  Within a step all of that is the same for every
layer of one kind; only the addresses of the layer's own tensors differ.  So the first
layer of a kind that meets a given kind of input runs as written while its launches are
listed (``kernels.ops.recording``), and every later layer of that kind launches from the
list, with the addresses of its own weights, cache arrays, incoming sub-layer output and
following norm in place of the recorded layer's.  Everything else the recorded layer
allocated is kept until the step ends and used again: layers run one after the other on
one stream, so a buffer a layer has finished with is free for the next.

A block takes part only if it says ``replayable``: its parts launch all their work through
``kernels.ops`` and decide nothing from values that differ between layers of a kind.
"""

from __future__ import annotations

import bisect
import dataclasses
from ctypes import c_void_p
from dataclasses import dataclass, field

import numpy as np
import torch

from tokamak_amd.kernels import ops
from tokamak_amd.kernels.linear import Added


def _span_bytes(t: torch.Tensor) -> int:
    if t.numel() == 0:
        return 0
    return (sum((size - 1) * stride for size, stride in zip(t.shape, t.stride())) + 1) * t.element_size()


def _fields(obj) -> list[tuple[str, torch.Tensor]]:
    """The GPU tensors an object holds as attributes."""
    return [(name, value) for name, value in vars(obj).items() if isinstance(value, torch.Tensor) and value.is_cuda]


def pending_tensors(pending) -> list[tuple[str, torch.Tensor]]:
    if pending is None:
        return []
    if isinstance(pending, torch.Tensor):
        return [("", pending)]
    return _fields(pending)


def pending_kind(pending) -> tuple:
    """What must agree between the recorded layer's incoming sub-layer output and another's."""
    return (type(pending).__name__, tuple((name, tuple(t.shape), t.dtype, t.stride()) for name, t in pending_tensors(pending)))


def _stores(store) -> list[tuple[str, object]]:
    """(role, slot store) pairs of what a block receives as ``store``: one slot, or a dict of
    slots by the roles of its mixers."""
    return list(store.items()) if isinstance(store, dict) else [("", store)]


def store_groups(store) -> tuple[int, ...]:
    return tuple(s.group for _, s in _stores(store))


def own_tensors(block, store) -> dict[tuple, torch.Tensor]:
    """The tensors that belong to one layer call: its parts' and its cache slots'."""
    out: dict[tuple, torch.Tensor] = {}
    for role, part in block.parts.items():
        for name, t in _fields(part):
            out[("part", role, name)] = t
    for role, slot in _stores(store):
        for name, t in slot.arrays.items():
            out[("cache", role, name)] = t
        for name, t in slot.state.items():
            out[("state", role, name)] = t
    return out


def call_tensors(own: dict, pending, then) -> dict[tuple, torch.Tensor]:
    out = dict(own)
    for name, t in pending_tensors(pending):
        out[("pending", name)] = t
    if then is not None:
        for name, t in _fields(then):
            out[("then", name)] = t
    return out


class PackedCalls:
    """A recording's calls laid out for ``ops.replay_calls``: the slot forms' addresses, every
    call's arguments as 64-bit slots in one array, and the patches (slot, index of the tensor
    in ``keys``, offset inside it).  One foreign call then issues a whole layer."""

    def __init__(self, calls: list[tuple]) -> None:
        fns, first, slots, expected = [], [], [], []
        patch_slot, patch_key, patch_offset = [], [], []
        self.keys: list[tuple] = []
        index: dict[tuple, int] = {}
        self.ok = True
        for fn, args, patches, status in calls:
            packed = ops.slots_of(fn, args)
            if packed is None:
                self.ok = False
                return
            fns.append(fn.slots_address)
            first.append(len(slots))
            for at, key, offset in patches:
                if key not in index:
                    index[key] = len(self.keys)
                    self.keys.append(key)
                patch_slot.append(len(slots) + at)
                patch_key.append(index[key])
                patch_offset.append(offset)
            slots.extend(packed)
            expected.append(status)
        self.fns = np.array(fns, dtype=np.uint64)
        self.first = np.array(first, dtype=np.int32)
        self.slots = np.array(slots, dtype=np.uint64)
        self.expected = np.array(expected, dtype=np.int32)
        self.patch_slot = np.array(patch_slot, dtype=np.int32)
        self.patch_key = np.array(patch_key, dtype=np.int32)
        self.patch_offset = np.array(patch_offset, dtype=np.int64)
        self.addresses = np.zeros(max(1, len(self.keys)), dtype=np.uint64)
        self.got = np.zeros(1, dtype=np.int32)
        self.pointers = tuple(a.ctypes.data for a in (self.fns, self.first, self.slots))
        self.patch_pointers = tuple(a.ctypes.data for a in (self.patch_slot, self.patch_key, self.patch_offset,
                                                            self.addresses, self.expected, self.got))

    def launch(self, tensors: dict[tuple, torch.Tensor]) -> None:
        addresses = self.addresses
        for i, key in enumerate(self.keys):
            addresses[i] = tensors[key].data_ptr()
        bad = ops.replay_calls(len(self.expected), *self.pointers, len(self.patch_slot), *self.patch_pointers)
        if bad >= 0:
            raise ops.KernelError(f"replayed launch {bad} returned {int(self.got[0])}, the recorded one "
                                  f"{int(self.expected[bad])}")


@dataclass
class LayerRecording:
    """The list is packed for the one-call form after its first replay, not when it is made:
    the first layers of a step are launched while the GPU has nothing else to do, and the
    packing (some 0.1 ms) would hold up the second layer's kernels; after it, the GPU has that
    layer's work and the host's time is hidden (a step of 2,048 tokens at 0.6B width, timed
    from an idle GPU: 5.46 ms packed at once, 5.36 never packed or packed after the first replay)."""

    calls: list[tuple]          # (function, arguments, ((argument index, tensor key, byte offset), ...), status)
    keep: list[torch.Tensor]
    result: object
    packed: PackedCalls | None = field(default=None, repr=False)
    pack_tried: bool = field(default=False, repr=False)

    def launch(self, tensors: dict[tuple, torch.Tensor], then):
        if self.packed is not None:
            self.packed.launch(tensors)         # the whole layer in one foreign call
        else:
            address = {key: t.data_ptr() for key, t in tensors.items()}     # once a layer, not once a patch
            for fn, args, patches, status in self.calls:
                if patches:
                    args = list(args)
                    for index, key, offset in patches:
                        args[index] = address[key] + offset     # a plain int is taken for a pointer argument
                got = fn(*args)
                if got != status:
                    raise ops.KernelError(f"a replayed launch returned {got}, the recorded one {status}")
            if not self.pack_tried:
                self.pack_tried = True
                packed = PackedCalls(self.calls)
                self.packed = packed if packed.ok else None
        result = self.result
        if isinstance(result, Added) and result.gamma is not None:
            # the stream times the weight of the norm that follows THIS layer
            result = dataclasses.replace(result, gamma=then.sink(None).gamma)
        return result


def record(run, tensors: dict[tuple, torch.Tensor]):
    """Run ``run()`` while its launches are listed.  Returns (its result, a LayerRecording or
    None if what ran cannot be replayed)."""
    with ops.recording() as recorder:
        result = run()
    if not recorder.valid:
        return result, None
    spans = sorted((t.data_ptr(), t.data_ptr() + _span_bytes(t), key) for key, t in tensors.items() if t.numel())
    starts = [s[0] for s in spans]
    calls = []
    for fn, args, status in recorder.calls:
        patches = []
        for index, arg in enumerate(args):
            if not isinstance(arg, c_void_p) or not arg.value:
                continue
            at = bisect.bisect_right(starts, arg.value) - 1     # (the spans of different tensors do not overlap)
            if at >= 0 and spans[at][0] <= arg.value < spans[at][1]:
                patches.append((index, spans[at][2], arg.value - spans[at][0]))
        calls.append((fn, args, tuple(patches), status))
    return result, LayerRecording(calls, recorder.keep, result)
