"""Layer-offload streaming of packed GGUF weights on HIP.

Keeps the tensors of every layer of an ``nn.ModuleList`` in pinned host memory and brings them onto
the GPU for the layer's forward, optionally ahead of time on a second stream.  Interface and
semantics follow the reference's layer offloader
(``src/sensenova_u1/utils/layer_offload.py``: tensor groups ``:51-54``, tower partition ``:195-222``,
group selection from the layer kwargs ``:225-241``, store ``:289-419``; what the prefetcher ``:422-462`` and the
hooks ``:764-843`` of the wrapper ``:465-999`` achieve is reached differently), the data movement does not:

* every (layer, group) is packed once into ONE contiguous pinned arena, so bringing a tower of a
  layer onto the GPU is a single asynchronous copy of ~100-200 MB instead of one copy per tensor,
  and ``tensor.data`` is rebound to views of that arena (host) or of a device slot;
* device memory is a small ring of slots per group (as many as are in flight: one plus the
  prefetch depth), allocated on first use and then reused for the rest of the process, so a
  forward pass allocates nothing and no caching-allocator stream bookkeeping (``record_stream``)
  is involved.  A slot carries the event recorded on the compute stream when its layer was evicted;
  the stream that next copies into the slot waits for that event first;
* copying ahead is part of the store (``copy_ahead`` / ``make_ready``): a copy on the store's second stream leaves
  a "landed" event with the slot, the consumer's stream waits for it, and a slot handed back before anyone consumed
  its copy takes that event along to its next user.  A change of tower therefore needs no device-wide
  synchronisation: the slots of the tower that is no longer read simply go back to the ring.

The VRAM-budget residency policy, the prefix/denoise phase callback and the diagnostics of the
reference wrapper (``:68-116,684-762,863-919``) are control plane and are not rebuilt; the only
residency option kept is ``keep_generation_resident`` with an explicit byte budget.
"""
from __future__ import annotations

import itertools
from typing import Any, Optional

import torch
from torch import nn

GROUP_SHARED = "shared"
GROUP_UNDERSTANDING = "understanding"
GROUP_GENERATION = "generation"
ALL_TENSOR_GROUPS = frozenset({GROUP_SHARED, GROUP_UNDERSTANDING, GROUP_GENERATION})
_GEN_SUFFIX = "_mot_gen"
_ALIGN = 256  # arena offsets: a multiple of every element size and of the kernels' 16-byte row alignment


def partition_layer_tensor_names(layer: nn.Module) -> dict[str, str]:
    """Tensor name -> group.  A tensor under a module path component ending in ``_mot_gen`` belongs to the
    generation tower; a tensor that has such a twin belongs to the understanding tower; everything else
    (norm-free buffers, layers without towers) is shared (reference ``layer_offload.py:195-222``)."""
    names = {n for n, _ in itertools.chain(layer.named_parameters(), layer.named_buffers())}
    out: dict[str, str] = {}
    for name in names:
        parts = name.split(".")
        owners = parts[:-1]
        if any(p.endswith(_GEN_SUFFIX) for p in owners):
            out[name] = GROUP_GENERATION
            continue
        twin = any(".".join(parts[:i] + [parts[i] + _GEN_SUFFIX] + parts[i + 1:]) in names for i in range(len(owners)))
        out[name] = GROUP_UNDERSTANDING if twin else GROUP_SHARED
    return out


def required_tensor_groups(kwargs: dict[str, Any]) -> frozenset[str]:
    """Groups one decoder-layer call needs, from its two tower flags; anything but two Python bools
    means all groups (reference ``layer_offload.py:225-241``)."""
    und = kwargs.get("exist_non_image_gen_tokens")
    gen = kwargs.get("exist_image_gen_tokens")
    if not isinstance(und, bool) or not isinstance(gen, bool) or und == gen:
        return ALL_TENSOR_GROUPS
    return frozenset({GROUP_SHARED, GROUP_UNDERSTANDING if und else GROUP_GENERATION})


def _round_up(v: int, a: int) -> int:
    return (v + a - 1) // a * a


class _Arena:
    """The tensors of one (layer, group), packed back to back in one host buffer."""

    __slots__ = ("host", "entries", "nbytes")

    def __init__(self, tensors: list[tuple[str, torch.Tensor]], pin_memory: bool) -> None:
        self.entries: list[tuple[torch.Tensor, int, int, torch.dtype, tuple]] = []
        off = 0
        for _name, t in tensors:
            n = t.numel() * t.element_size()
            self.entries.append((t, off, n, t.dtype, tuple(t.shape)))
            off = _round_up(off + n, _ALIGN)
        self.nbytes = off
        self.host = torch.empty(off, dtype=torch.uint8, pin_memory=pin_memory)
        for t, o, n, _dt, _shape in self.entries:
            if n:
                self.host[o:o + n].copy_(t.data.detach().contiguous().reshape(-1).view(torch.uint8).cpu())
        self.bind(self.host)

    def bind(self, buf: torch.Tensor) -> None:
        """Point every tensor's ``.data`` at its slice of ``buf`` (the host arena or a device slot)."""
        for t, o, n, dt, shape in self.entries:
            t.data = buf[o:o + n].view(dt).view(shape)


class PackedLayerStore:
    """Pinned arenas for every layer of ``layers`` plus the ring of device slots they are copied into.

    Same bookkeeping interface as the reference store (``layer_offload.py:289-419``): ``is_on_gpu``,
    ``move_to_gpu``, ``evict_to_cpu``, ``tensors_for_groups``, ``transfer_stats``, ``group_nbytes``,
    ``managed_tensor_ids``, ``cleanup``.  ``move_to_gpu`` enqueues on the CURRENT stream; eviction drops no
    memory, it returns the slot to the ring together with an event on the current stream.
    """

    def __init__(self, layers, target_device: torch.device, pin_memory: bool = True) -> None:
        self.target_device = torch.device(target_device)
        self.num_layers = len(layers)
        self._arenas: list[dict[str, _Arena]] = []
        self._tensor_groups: list[dict[str, str]] = []
        self._resident: list[dict[str, torch.Tensor]] = []
        self._managed: set[int] = set()
        # free slots, each with the events its next user must wait for: the compute-stream event of the eviction and,
        # if a copy into it was still unconsumed at that point, that copy's event
        self._free: dict[str, list[tuple[torch.Tensor, list]]] = {g: [] for g in ALL_TENSOR_GROUPS}
        self._ready: list[dict[str, Any]] = []      # per layer: group -> event of a copy-ahead nobody has waited for yet
        self._copy_stream = None
        self._slot_bytes = {g: 0 for g in ALL_TENSOR_GROUPS}
        self._slots_allocated = {g: 0 for g in ALL_TENSOR_GROUPS}
        self._bytes_moved = 0
        self._bytes_moved_by_group = {g: 0 for g in ALL_TENSOR_GROUPS}
        self._copies = 0
        # A tensor that several layers share cannot follow one layer in and out: it is left unmanaged, which
        # the wrapper treats like everything outside the layer list (resident on the device).
        seen: dict[int, int] = {}
        for layer in layers:
            for _name, t in itertools.chain(layer.named_parameters(), layer.named_buffers()):
                seen[id(t)] = seen.get(id(t), 0) + 1
        for layer in layers:
            groups = partition_layer_tensor_names(layer)
            by_group: dict[str, list[tuple[str, torch.Tensor]]] = {}
            for name, t in itertools.chain(layer.named_parameters(), layer.named_buffers()):
                if seen[id(t)] > 1:
                    continue
                self._managed.add(id(t))
                by_group.setdefault(groups.get(name, GROUP_SHARED), []).append((name, t))
            arenas = {g: _Arena(ts, pin_memory) for g, ts in by_group.items()}
            # q / k / v that a loader stacked into one device tensor now live in the arenas: the stack lets go of its copy
            for mod in layer.modules():
                stack = mod.__dict__.get("_shared_stack")
                if stack is not None:
                    stack.release_if_moved()
            for g, a in arenas.items():
                self._slot_bytes[g] = max(self._slot_bytes[g], a.nbytes)
            self._arenas.append(arenas)
            self._tensor_groups.append(groups)
            self._resident.append({})
            self._ready.append({})

    def _check_idx(self, idx: int) -> None:
        if idx < 0 or idx >= self.num_layers:
            raise IndexError(f"Layer index {idx} out of range [0, {self.num_layers})")

    def is_on_gpu(self, idx: int, groups: Optional[frozenset] = None) -> bool:
        self._check_idx(idx)
        have = self._resident[idx]
        if groups is None:
            return bool(have)
        return all(g in have or g not in self._arenas[idx] for g in groups)

    def _take_slot(self, group: str) -> torch.Tensor:
        if self._free[group]:
            slot, events = self._free[group].pop()
            for event in events:
                torch.cuda.current_stream(self.target_device).wait_event(event)
            return slot
        self._slots_allocated[group] += 1
        return torch.empty(max(self._slot_bytes[group], _ALIGN), dtype=torch.uint8, device=self.target_device)

    def move_to_gpu(self, idx: int, layer: nn.Module = None, *, groups: frozenset = ALL_TENSOR_GROUPS,
                    non_blocking: bool = False) -> None:
        """One copy per missing group of layer ``idx`` into a ring slot, on the current stream."""
        self._check_idx(idx)
        have = self._resident[idx]
        for g in sorted(groups):
            arena = self._arenas[idx].get(g)
            if arena is None or g in have:
                continue
            slot = self._take_slot(g)
            if arena.nbytes:
                slot[:arena.nbytes].copy_(arena.host, non_blocking=non_blocking)
            arena.bind(slot)
            have[g] = slot
            self._bytes_moved += arena.nbytes
            self._bytes_moved_by_group[g] += arena.nbytes
            self._copies += 1

    def evict_to_cpu(self, idx: int, layer: nn.Module = None, *, groups: frozenset = ALL_TENSOR_GROUPS) -> None:
        """Rebind the tensors to their pinned arena and hand the slots back; work already enqueued on
        the current stream may still read them, which the slot's event covers."""
        self._check_idx(idx)
        have = self._resident[idx]
        for g in sorted(groups):
            slot = have.pop(g, None)
            if slot is None:
                continue
            self._arenas[idx][g].bind(self._arenas[idx][g].host)
            events = []
            if self.target_device.type == "cuda":
                done = torch.cuda.Event()
                done.record(torch.cuda.current_stream(self.target_device))
                events.append(done)
            unconsumed = self._ready[idx].pop(g, None)
            if unconsumed is not None:
                events.append(unconsumed)
            self._free[g].append((slot, events))

    # ---- copy-ahead on a second stream: the slot ring's events are the whole protocol -------------------------------
    # A slot goes round as: free (carrying the events of its last use) -> copy target (the copying stream waits for
    # those events) -> resident, perhaps with a "ready" event from the copy stream -> in use (the consumer waited for
    # the ready event) -> free again.  No stream is ever synchronised with the host.

    def copy_ahead(self, idx: int, groups: frozenset) -> None:
        """Start bringing the missing groups of layer ``idx`` in on the store's copy stream (created on first use,
        default priority).  Returns at once; ``make_ready`` later orders a consumer stream behind the copy."""
        self._check_idx(idx)
        missing = frozenset(g for g in groups if g in self._arenas[idx] and g not in self._resident[idx])
        if not missing:
            return
        if self._copy_stream is None:
            self._copy_stream = torch.cuda.Stream(device=self.target_device)
        with torch.cuda.stream(self._copy_stream):
            self.move_to_gpu(idx, groups=missing, non_blocking=True)
            landed = torch.cuda.Event()
            landed.record(self._copy_stream)
        for g in missing:
            self._ready[idx][g] = landed

    def make_ready(self, idx: int, groups: frozenset) -> None:
        """After this call, work enqueued on the current stream may read ``groups`` of layer ``idx``: copies started by
        ``copy_ahead`` are waited for (on the stream, not on the host), anything still missing is copied on the
        current stream itself."""
        self._check_idx(idx)
        stream = torch.cuda.current_stream(self.target_device) if self.target_device.type == "cuda" else None
        waited: set[int] = set()
        for g in groups:
            landed = self._ready[idx].pop(g, None)
            if landed is not None and id(landed) not in waited:
                stream.wait_event(landed)
                waited.add(id(landed))
        self.move_to_gpu(idx, groups=groups, non_blocking=True)

    def copies_in_flight(self) -> set[int]:
        """Layers with a copy-ahead that no consumer has been ordered behind yet."""
        return {i for i, r in enumerate(self._ready) if r}

    def tensors_for_groups(self, idx: int, layer: nn.Module, groups: frozenset) -> list[torch.Tensor]:
        self._check_idx(idx)
        tg = self._tensor_groups[idx]
        return [t for name, t in itertools.chain(layer.named_parameters(), layer.named_buffers())
                if tg.get(name, GROUP_SHARED) in groups]

    def transfer_stats(self) -> tuple[int, dict[str, int]]:
        return self._bytes_moved, dict(self._bytes_moved_by_group)

    def copies_issued(self) -> int:
        return self._copies

    def group_nbytes(self, idx: int, group: str) -> int:
        """Bytes of the tensors of one group of a layer (without alignment padding)."""
        self._check_idx(idx)
        arena = self._arenas[idx].get(group)
        return 0 if arena is None else sum(n for _t, _o, n, _dt, _s in arena.entries)

    def device_bytes(self) -> int:
        """Device memory held by the slot ring, in use or free."""
        return sum(self._slots_allocated[g] * max(self._slot_bytes[g], _ALIGN) for g in ALL_TENSOR_GROUPS)

    def slots_allocated(self) -> dict[str, int]:
        return dict(self._slots_allocated)

    def managed_tensor_ids(self) -> set[int]:
        return set(self._managed)

    def cleanup(self) -> None:
        """Evict everything and drop the device ring (after the device has finished with it).  Tensors keep
        their pinned arena views."""
        if self.target_device.type == "cuda":
            torch.cuda.synchronize(self.target_device)
        for idx in range(self.num_layers):
            self.evict_to_cpu(idx)
        for g in self._free:
            self._free[g].clear()
            self._slots_allocated[g] = 0
        self._copy_stream = None


def _layer_list(model: nn.Module, dotted: str) -> nn.ModuleList:
    found = model.get_submodule(dotted) if dotted else model
    if not isinstance(found, nn.ModuleList):
        raise TypeError(f"'{dotted}' is a {type(found).__name__}; layer streaming needs an nn.ModuleList")
    return found


class LayerStreamer:
    """Installs layer streaming on a model in place: every layer of the list gets a gate in front of its forward
    (bring my groups in, start the copies for the layers after me) and one behind it (hand my slots back).

    The model stays the callable; this object only owns the store, the schedule and the hook handles.
    """

    def __init__(self, model: nn.Module, layers: nn.ModuleList, target_device: torch.device, depth: int,
                 keep_generation_resident: bool, resident_budget_bytes: Optional[int]) -> None:
        self.model = model
        self.layers = layers
        self.device = target_device
        self.depth = min(depth, max(len(layers) - 1, 0))
        self.keep_generation = keep_generation_resident
        self.budget = resident_budget_bytes
        self.store = PackedLayerStore(layers, target_device)
        managed = self.store.managed_tensor_ids()
        self._outside = [t for t in itertools.chain(model.parameters(), model.buffers()) if id(t) not in managed]
        for t in self._outside:
            t.data = t.data.to(target_device)
        self._tower: Optional[frozenset] = None       # groups of the call in progress / the last call
        self._in_forward: dict[int, frozenset] = {}
        self._handles = []
        for idx, layer in enumerate(layers):
            self._handles.append(layer.register_forward_pre_hook(self._gate_in(idx), with_kwargs=True))
            self._handles.append(layer.register_forward_hook(self._gate_out(idx)))

    # -- schedule ---------------------------------------------------------------------------------------------------
    def _upcoming(self, idx: int):
        """The layers whose copies should be under way while layer ``idx`` runs: the next ``depth`` ones, wrapping
        round to the first layers, which the next pass over the list starts with."""
        n = len(self.layers)
        return [(idx + step) % n for step in range(1, self.depth + 1)]

    def _retarget(self, groups: frozenset) -> None:
        """The call reads other groups than the last one did: slots holding a group it does not read go back to the
        ring (their events keep work in flight safe), except a generation tower that is being kept."""
        stale = ALL_TENSOR_GROUPS - groups
        if self.keep_generation and self._within_budget():
            stale = stale - {GROUP_GENERATION}
        if stale and self._tower is not None:
            for idx in range(len(self.layers)):
                self.store.evict_to_cpu(idx, groups=stale)
        self._tower = groups

    def _within_budget(self) -> bool:
        return self.budget is None or self.store.device_bytes() <= self.budget

    def _gate_in(self, idx: int):
        def gate(layer, args, kwargs):
            groups = required_tensor_groups(kwargs)
            if groups != self._tower:
                self._retarget(groups)
            self.store.make_ready(idx, groups)
            for nxt in self._upcoming(idx):
                self.store.copy_ahead(nxt, groups)
            self._in_forward[idx] = groups
        return gate

    def _gate_out(self, idx: int):
        def gate(layer, args, output):
            groups = self._in_forward.pop(idx, ALL_TENSOR_GROUPS)
            if self.keep_generation and GROUP_GENERATION in groups and self._within_budget():
                groups = groups - {GROUP_GENERATION}
            self.store.evict_to_cpu(idx, groups=groups)
        return gate

    def remove(self) -> None:
        """Take the gates off, wait for the device, put every tensor back on the host (layer tensors in their pinned
        arenas) and drop the slot ring."""
        for h in self._handles:
            h.remove()
        self._handles = []
        self.store.cleanup()
        for t in self._outside:
            t.data = t.data.to("cpu")


class LayerOffloadWrapper(nn.Module):
    """``model`` with the layers of ``layers_attr`` streamed from pinned host memory; same constructor arguments and
    use as the reference's wrapper (``layer_offload.py:501-530``): call it like the model, read the model's attributes
    through it, ``teardown()`` when done.

    ``prefetch_count == 0``: a layer's groups are copied on the compute stream right before its forward; ``>= 1``:
    that many layers ahead are copied on a second stream, wrapping around to the first layers for the next pass.
    Only the groups a call needs are brought in, chosen from the layer kwargs ``exist_non_image_gen_tokens`` /
    ``exist_image_gen_tokens``.  Everything outside ``layers_attr`` is moved to ``target_device`` once and stays
    there.  Inference only.  The work is done by :class:`LayerStreamer` (``.streamer``).
    """

    def __init__(self, model: nn.Module, layers_attr: str, target_device: torch.device, prefetch_count: int = 0,
                 keep_generation_resident: bool = False, resident_budget_bytes: Optional[int] = None) -> None:
        super().__init__()
        target_device = torch.device(target_device)
        if target_device.type != "cuda":
            raise ValueError(f"LayerOffloadWrapper needs a GPU target device, got {target_device}")
        if prefetch_count < 0:
            raise ValueError("prefetch_count must be >= 0")
        if resident_budget_bytes is not None and resident_budget_bytes <= 0:
            raise ValueError("resident_budget_bytes must be > 0 when set")
        if model.training:
            raise RuntimeError("LayerOffloadWrapper only supports inference; call model.eval() first.")
        layers = _layer_list(model, layers_attr)
        self.wrapped = model
        # (a plain attribute, not a submodule: the streamer refers back to the model)
        object.__setattr__(self, "streamer", LayerStreamer(model, layers, target_device, prefetch_count,
                                                           keep_generation_resident, resident_budget_bytes))

    @property
    def store(self) -> PackedLayerStore:
        return self.streamer.store

    def transfer_stats(self) -> tuple[int, dict[str, int]]:
        return self.streamer.store.transfer_stats()

    def teardown(self) -> None:
        self.streamer.remove()

    def forward(self, *args: Any, **kwargs: Any) -> Any:
        return self.wrapped(*args, **kwargs)

    def __getattr__(self, name: str) -> Any:
        # nn.Module keeps submodules out of __dict__; anything this wrapper does not have is the model's
        modules = self.__dict__.get("_modules", {})
        if name in modules:
            return modules[name]
        if "wrapped" in modules:
            return getattr(modules["wrapped"], name)
        raise AttributeError(name)
