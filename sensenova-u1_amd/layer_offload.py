"""Layer-offload streaming of packed GGUF weights on HIP.

Keeps the tensors of every layer of an ``nn.ModuleList`` in pinned host memory and brings them onto
the GPU for the layer's forward, optionally ahead of time on a second stream.  Interface and
semantics follow the reference's layer offloader
(``src/sensenova_u1/utils/layer_offload.py``: tensor groups ``:51-54``, tower partition ``:195-222``,
group selection from the layer kwargs ``:225-241``, store ``:289-419``, prefetcher ``:422-462``,
hooks ``:764-843``, wrapper ``:465-999``), the data movement does not:

* every (layer, group) is packed once into ONE contiguous pinned arena, so bringing a tower of a
  layer onto the GPU is a single asynchronous copy of ~100-200 MB instead of one copy per tensor,
  and ``tensor.data`` is rebound to views of that arena (host) or of a device slot;
* device memory is a small ring of slots per group (as many as are in flight: one plus the
  prefetch depth), allocated on first use and then reused for the rest of the process, so a
  forward pass allocates nothing and no caching-allocator stream bookkeeping (``record_stream``)
  is involved.  A slot carries the event recorded on the compute stream when its layer was evicted;
  the stream that next copies into the slot waits for that event first.

The VRAM-budget residency policy, the prefix/denoise phase callback and the diagnostics of the
reference wrapper (``:68-116,684-762,863-919``) are control plane and are not rebuilt; the only
residency option kept is ``keep_generation_resident`` with an explicit byte budget.
"""
from __future__ import annotations

import functools
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
        self._free: dict[str, list[tuple[torch.Tensor, Any]]] = {g: [] for g in ALL_TENSOR_GROUPS}
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
            for g, a in arenas.items():
                self._slot_bytes[g] = max(self._slot_bytes[g], a.nbytes)
            self._arenas.append(arenas)
            self._tensor_groups.append(groups)
            self._resident.append({})

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
            slot, event = self._free[group].pop()
            if event is not None:
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
            event = None
            if self.target_device.type == "cuda":
                event = torch.cuda.Event()
                event.record(torch.cuda.current_stream(self.target_device))
            self._free[g].append((slot, event))

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


class AsyncPrefetcher:
    """Copies upcoming layers on a second stream (default priority); one event per layer so the compute
    stream waits only for the layer it is about to run (reference ``layer_offload.py:422-462``)."""

    def __init__(self, store: PackedLayerStore, layers) -> None:
        self._store = store
        self._layers = layers
        self._stream = torch.cuda.Stream(device=store.target_device)
        self._events: dict[int, tuple[Any, frozenset]] = {}

    @property
    def stream(self):
        return self._stream

    def prefetch(self, idx: int, groups: frozenset) -> None:
        if self._store.is_on_gpu(idx, groups) or idx in self._events:
            return
        with torch.cuda.stream(self._stream):
            self._store.move_to_gpu(idx, self._layers[idx], groups=groups, non_blocking=True)
            event = torch.cuda.Event()
            event.record(self._stream)
        self._events[idx] = (event, groups)

    def wait(self, idx: int) -> None:
        pending = self._events.pop(idx, None)
        if pending is not None:
            torch.cuda.current_stream(self._store.target_device).wait_event(pending[0])

    def pending(self) -> set[int]:
        return set(self._events)

    def clear_events(self) -> None:
        self._events.clear()

    def cleanup(self) -> None:
        self._events.clear()
        self._stream = None
        self._layers = None
        self._store = None


def _resolve_attr(module: nn.Module, dotted_path: str) -> nn.ModuleList:
    obj: Any = module
    for part in dotted_path.split("."):
        obj = getattr(obj, part)
    if not isinstance(obj, nn.ModuleList):
        raise TypeError(f"Expected nn.ModuleList at '{dotted_path}', got {type(obj).__name__}")
    return obj


class LayerOffloadWrapper(nn.Module):
    """Runs ``model`` with the layers of ``layers_attr`` streamed from pinned host memory.

    ``prefetch_count == 0``: a layer's groups are copied on the compute stream right before its forward;
    ``>= 1``: that many layers ahead are copied on a second stream, wrapping around to the first layers
    for the next pass.  Only the groups a call needs are brought in, chosen from the layer kwargs
    ``exist_non_image_gen_tokens`` / ``exist_image_gen_tokens``.  Everything outside ``layers_attr`` is
    moved to ``target_device`` once and stays there.  Inference only.
    Constructor and behaviour after reference ``layer_offload.py:501-530,607-642,764-843,921-999``.
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
        self._model = model
        self._layers = _resolve_attr(model, layers_attr)
        self._target_device = target_device
        self._prefetch_count = min(prefetch_count, max(len(self._layers) - 1, 0))
        self._async_mode = self._prefetch_count >= 1
        self._keep_generation_resident = keep_generation_resident
        self._resident_budget_bytes = resident_budget_bytes
        self._active_groups: Optional[frozenset] = None
        self._hooks: list = []
        self._store = PackedLayerStore(self._layers, target_device)
        managed = self._store.managed_tensor_ids()
        for t in itertools.chain(model.parameters(), model.buffers()):
            if id(t) not in managed:
                t.data = t.data.to(target_device)
        self._prefetcher = AsyncPrefetcher(self._store, self._layers) if self._async_mode else None
        self._register_hooks()

    @property
    def store(self) -> PackedLayerStore:
        return self._store

    def _switch_groups(self, groups: frozenset) -> None:
        """A change of tower drains the copy stream and evicts what the other tower left behind."""
        if self._active_groups == groups:
            return
        if self._active_groups is not None:
            torch.cuda.synchronize(self._target_device)
            if self._prefetcher is not None:
                self._prefetcher.clear_events()
            for idx, layer in enumerate(self._layers):
                self._store.evict_to_cpu(idx, layer)
        self._active_groups = groups

    def _groups_to_evict(self, idx: int, groups: frozenset) -> frozenset:
        if not self._keep_generation_resident or GROUP_GENERATION not in groups:
            return groups
        if self._resident_budget_bytes is not None and self._store.device_bytes() > self._resident_budget_bytes:
            return groups
        return groups - {GROUP_GENERATION}

    def _register_hooks(self) -> None:
        num_layers = len(self._layers)
        active: dict[int, frozenset] = {}

        def pre_hook(module, args, kwargs, *, idx: int) -> None:
            groups = required_tensor_groups(kwargs)
            active[idx] = groups
            self._switch_groups(groups)
            if self._async_mode:
                self._prefetcher.wait(idx)
                if not self._store.is_on_gpu(idx, groups):
                    self._store.move_to_gpu(idx, module, groups=groups, non_blocking=True)
                for ahead in range(1, self._prefetch_count + 1):
                    self._prefetcher.prefetch((idx + ahead) % num_layers, groups)
            else:
                self._store.move_to_gpu(idx, module, groups=groups, non_blocking=True)

        def post_hook(module, _args, _output, *, idx: int) -> None:
            groups = active.pop(idx, ALL_TENSOR_GROUPS)
            self._store.evict_to_cpu(idx, module, groups=self._groups_to_evict(idx, groups))

        for idx, layer in enumerate(self._layers):
            self._hooks.append(layer.register_forward_pre_hook(functools.partial(pre_hook, idx=idx), with_kwargs=True))
            self._hooks.append(layer.register_forward_hook(functools.partial(post_hook, idx=idx)))

    def transfer_stats(self) -> tuple[int, dict[str, int]]:
        return self._store.transfer_stats()

    def teardown(self) -> None:
        """Remove the hooks, drain the copies, leave every tensor on the host (layer tensors in their
        pinned arenas) and release the device ring."""
        for h in self._hooks:
            h.remove()
        self._hooks.clear()
        torch.cuda.synchronize(self._target_device)
        if self._prefetcher is not None:
            self._prefetcher.cleanup()
            self._prefetcher = None
        self._store.cleanup()
        managed = self._store.managed_tensor_ids()
        for t in itertools.chain(self._model.parameters(), self._model.buffers()):
            if id(t) not in managed:
                t.data = t.data.to("cpu")

    def forward(self, *args: Any, **kwargs: Any) -> Any:
        return self._model(*args, **kwargs)

    def __getattr__(self, name: str) -> Any:
        try:
            return super().__getattr__(name)
        except AttributeError:
            return getattr(self._model, name)
