"""Host logic of the layer-offload streaming (no GPU): tower partition and group selection with the
cases the reference's own tests pin (tests/test_layer_offload.py:267-303 of the reference), arena packing
and the slot ring with the "device" being the CPU."""
import pytest
import torch
from torch import nn

from sensenova_u1_amd import GGUFLinear, GGUFParameter, synthetic
from sensenova_u1_amd.layer_offload import (ALL_TENSOR_GROUPS, GROUP_GENERATION, GROUP_SHARED, GROUP_UNDERSTANDING,
                                            LayerOffloadWrapper, PackedLayerStore, partition_layer_tensor_names,
                                            required_tensor_groups)

H, I = 256, 512


def _q(n, k, seed, qt=8):
    lin = GGUFLinear(k, n, bias=False, compute_dtype=torch.bfloat16)
    lin.weight = GGUFParameter(synthetic.make_packed(qt, n, k, seed=seed), quant_type=qt)
    return lin


class TwoTowerLayer(nn.Module):
    """Decoder-layer-shaped toy: paired projections, a paired norm, one shared buffer."""

    def __init__(self, seed=0):
        super().__init__()
        self.self_attn = nn.Module()
        self.self_attn.q_proj = _q(H, H, seed + 1)
        self.self_attn.q_proj_mot_gen = _q(H, H, seed + 2, qt=12)
        self.mlp = nn.Module()
        self.mlp.up_proj = _q(I, H, seed + 3)
        self.mlp_mot_gen = nn.Module()
        self.mlp_mot_gen.up_proj = _q(I, H, seed + 4, qt=14)
        self.norm = nn.LayerNorm(H)
        self.norm_mot_gen = nn.LayerNorm(H)
        self.register_buffer("shared_scale", torch.full((3,), float(seed)))


def test_partition_pairs_towers_and_leaves_the_rest_shared():
    g = partition_layer_tensor_names(TwoTowerLayer())
    assert g["self_attn.q_proj.weight"] == GROUP_UNDERSTANDING
    assert g["self_attn.q_proj_mot_gen.weight"] == GROUP_GENERATION
    assert g["mlp.up_proj.weight"] == GROUP_UNDERSTANDING
    assert g["mlp_mot_gen.up_proj.weight"] == GROUP_GENERATION
    assert g["norm.bias"] == GROUP_UNDERSTANDING and g["norm_mot_gen.bias"] == GROUP_GENERATION
    assert g["shared_scale"] == GROUP_SHARED


def test_partition_of_a_plain_layer_is_all_shared():
    g = partition_layer_tensor_names(nn.Sequential(nn.Linear(4, 8), nn.Linear(8, 4)))
    assert g and set(g.values()) == {GROUP_SHARED}


def test_a_suffix_on_the_tensor_name_itself_is_not_a_tower():
    layer = nn.Module()
    layer.register_buffer("scale_mot_gen", torch.ones(2))
    assert partition_layer_tensor_names(layer) == {"scale_mot_gen": GROUP_SHARED}


def test_group_selection_from_layer_kwargs():
    und = required_tensor_groups({"exist_non_image_gen_tokens": True, "exist_image_gen_tokens": False})
    gen = required_tensor_groups({"exist_non_image_gen_tokens": False, "exist_image_gen_tokens": True})
    assert und == frozenset({GROUP_SHARED, GROUP_UNDERSTANDING})
    assert gen == frozenset({GROUP_SHARED, GROUP_GENERATION})
    assert required_tensor_groups({"exist_non_image_gen_tokens": True, "exist_image_gen_tokens": True}) == ALL_TENSOR_GROUPS
    assert required_tensor_groups({}) == ALL_TENSOR_GROUPS
    # tensors instead of Python bools: the caller is unknown, take everything
    assert required_tensor_groups({"exist_non_image_gen_tokens": torch.tensor(False),
                                   "exist_image_gen_tokens": torch.tensor(True)}) == ALL_TENSOR_GROUPS


def _snapshot(layers):
    return [{n: t.detach().clone() for n, t in list(l.named_parameters()) + list(l.named_buffers())} for l in layers]


def _same(layers, snap):
    for l, s in zip(layers, snap):
        for n, t in list(l.named_parameters()) + list(l.named_buffers()):
            assert t.dtype == s[n].dtype and t.shape == s[n].shape
            assert torch.equal(t.detach().view(torch.uint8), s[n].view(torch.uint8)), n


def test_store_packs_each_group_into_one_arena_and_keeps_values_types_and_tags():
    layers = nn.ModuleList([TwoTowerLayer(0), TwoTowerLayer(10)])
    snap = _snapshot(layers)
    store = PackedLayerStore(layers, torch.device("cpu"), pin_memory=False)
    _same(layers, snap)
    w = layers[0].self_attn.q_proj.weight
    assert isinstance(w, GGUFParameter) and w.quant_type == 8 and w.dtype == torch.uint8
    assert layers[1].mlp_mot_gen.up_proj.weight.quant_type == 14
    # the tensors of a group are slices of one buffer, 256-byte aligned
    a = layers[0].self_attn.q_proj.weight.data
    b = layers[0].mlp.up_proj.weight.data
    assert a.untyped_storage().data_ptr() == b.untyped_storage().data_ptr()
    base = a.untyped_storage().data_ptr()   # page-aligned when pinned or on the device
    assert all((t.data_ptr() - base) % 256 == 0 for t in (a, b, layers[0].norm.bias.data))
    assert a.untyped_storage().data_ptr() != layers[0].self_attn.q_proj_mot_gen.weight.data.untyped_storage().data_ptr()
    assert store.group_nbytes(0, GROUP_UNDERSTANDING) == H * (H // 32 * 34) + I * (H // 32 * 34) + 2 * H * 4
    assert store.group_nbytes(0, GROUP_SHARED) == 12
    ids = store.managed_tensor_ids()
    assert id(layers[0].self_attn.q_proj.weight) in ids and id(layers[1].shared_scale) in ids
    assert len(ids) == 2 * 9


def test_store_moves_only_the_requested_groups_and_reuses_slots():
    layers = nn.ModuleList([TwoTowerLayer(s) for s in (0, 10, 20)])
    snap = _snapshot(layers)
    store = PackedLayerStore(layers, torch.device("cpu"), pin_memory=False)
    und = frozenset({GROUP_SHARED, GROUP_UNDERSTANDING})
    host_ptr = layers[0].self_attn.q_proj.weight.data_ptr()
    assert not store.is_on_gpu(0) and not store.is_on_gpu(0, und)
    store.move_to_gpu(0, layers[0], groups=und)
    assert store.is_on_gpu(0, und) and not store.is_on_gpu(0, ALL_TENSOR_GROUPS) and store.is_on_gpu(0)
    assert layers[0].self_attn.q_proj.weight.data_ptr() != host_ptr          # now a slot view
    gen_ptr = layers[0].self_attn.q_proj_mot_gen.weight.data_ptr()
    _same(layers, snap)
    total, by_group = store.transfer_stats()
    assert by_group[GROUP_GENERATION] == 0 and by_group[GROUP_UNDERSTANDING] > 0 and total == sum(by_group.values())
    assert store.copies_issued() == 2
    store.move_to_gpu(0, layers[0], groups=und)                             # already there: nothing moves
    assert store.copies_issued() == 2
    store.evict_to_cpu(0, layers[0], groups=und)
    assert layers[0].self_attn.q_proj.weight.data_ptr() == host_ptr and not store.is_on_gpu(0)
    assert layers[0].self_attn.q_proj_mot_gen.weight.data_ptr() == gen_ptr  # the other tower was never touched
    # a pass over all layers, one at a time, needs one slot per group
    for _ in range(2):
        for i, l in enumerate(layers):
            store.move_to_gpu(i, l, groups=und)
            _same(layers, snap)
            store.evict_to_cpu(i, l, groups=und)
    assert store.slots_allocated() == {GROUP_SHARED: 1, GROUP_UNDERSTANDING: 1, GROUP_GENERATION: 0}
    # two layers in flight need two
    store.move_to_gpu(0, layers[0]); store.move_to_gpu(1, layers[1])
    _same(layers, snap)
    assert store.slots_allocated() == {GROUP_SHARED: 2, GROUP_UNDERSTANDING: 2, GROUP_GENERATION: 2}
    store.cleanup()
    _same(layers, snap)
    assert not any(store.is_on_gpu(i) for i in range(3))
    with pytest.raises(IndexError):
        store.is_on_gpu(3)


def test_tensors_shared_between_layers_are_left_to_the_caller():
    a, b = TwoTowerLayer(0), TwoTowerLayer(1)
    b.norm.weight = a.norm.weight
    layers = nn.ModuleList([a, b])
    store = PackedLayerStore(layers, torch.device("cpu"), pin_memory=False)
    ids = store.managed_tensor_ids()
    assert len(ids) == 16 and id(a.norm.weight) not in ids
    ptr = a.norm.weight.data_ptr()
    store.move_to_gpu(1, b)
    store.evict_to_cpu(1, b)
    assert b.norm.weight is a.norm.weight and a.norm.weight.data_ptr() == ptr


def test_wrapper_argument_checks():
    model = nn.Module()
    model.layers = nn.ModuleList([TwoTowerLayer()])
    model.eval()
    with pytest.raises(ValueError):
        LayerOffloadWrapper(model, "layers", torch.device("cpu"))
    with pytest.raises(ValueError):
        LayerOffloadWrapper(model, "layers", torch.device("cuda:0"), prefetch_count=-1)
    model.train()
    with pytest.raises(RuntimeError):
        LayerOffloadWrapper(model, "layers", torch.device("cuda:0"))
    model.eval()
    model.norm = nn.LayerNorm(4)
    with pytest.raises(TypeError):
        LayerOffloadWrapper(model, "norm", torch.device("cuda:0"))


def test_a_shared_input_stack_lets_go_of_its_copy_once_the_weights_have_moved():
    """modality.SharedInputStack keeps q / k / v rows in one tensor; when a store rebinds every member's weight.data to
    its own arena the stacked tensor has no user left and must not stay alive (the device check of the constructor is
    side-stepped here: the bookkeeping is the same on any device)."""
    from sensenova_u1_amd.modality import SharedInputStack

    mods = [_q(64, H, 1), _q(32, H, 2), _q(32, H, 3)]
    stack = object.__new__(SharedInputStack)
    stack.members, stack.index = mods, {id(m): i for i, m in enumerate(mods)}
    stack.splits = [m.out_features for m in mods]
    stack.offsets = [0, 64, 96]
    stack.row_bytes = mods[0].weight.shape[1]
    stack.stacked = torch.cat([m.weight.as_tensor() for m in mods], dim=0)
    stack._pending = None
    for m, off in zip(mods, stack.offsets):
        m.weight.data = stack.stacked[off:off + m.out_features]
        m.__dict__["_shared_stack"] = stack
    assert stack.intact() and not stack.release_if_moved() and stack.stacked is not None
    layer = nn.Module()
    layer.q_proj, layer.k_proj, layer.v_proj = mods
    store = PackedLayerStore([layer], torch.device("cpu"), pin_memory=False)
    assert stack.stacked is None and not stack.intact()
    assert not any("_shared_stack" in m.__dict__ for m in mods)
    assert all(id(m.weight) in store.managed_tensor_ids() for m in mods)
    # one member moved, the others still in place: nothing is released
    mods2 = [_q(64, H, 4), _q(32, H, 5)]
    st2 = object.__new__(SharedInputStack)
    st2.members, st2.index, st2.splits, st2.offsets = mods2, {id(m): i for i, m in enumerate(mods2)}, [64, 32], [0, 64]
    st2.row_bytes, st2._pending = mods2[0].weight.shape[1], None
    st2.stacked = torch.cat([m.weight.as_tensor() for m in mods2], dim=0)
    for m, off in zip(mods2, st2.offsets):
        m.weight.data = st2.stacked[off:off + m.out_features]
        m.__dict__["_shared_stack"] = st2
    mods2[1].weight.data = mods2[1].weight.data.clone()
    assert not st2.intact() and st2.stacked is not None and "_shared_stack" in mods2[0].__dict__
