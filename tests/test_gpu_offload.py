"""GPU: layers streamed from pinned host arenas give bit-identical results to the same model held
resident, in the synchronous mode and with one or two layers copied ahead on the second stream, for
either tower and across repeated passes (slot reuse); only the tower a call needs is copied."""
import copy

import pytest
import torch
from torch import nn

from sensenova_u1_amd import synthetic
from sensenova_u1_amd.layer_offload import (ALL_TENSOR_GROUPS, GROUP_GENERATION, GROUP_SHARED, GROUP_UNDERSTANDING,
                                            LayerOffloadWrapper)
from tests.test_layer_offload import H, TwoTowerLayer

pytestmark = pytest.mark.gpu


class Layer(TwoTowerLayer):
    def forward(self, h, exist_non_image_gen_tokens=None, exist_image_gen_tokens=None):
        gen = exist_image_gen_tokens is True and exist_non_image_gen_tokens is False
        attn = self.self_attn.q_proj_mot_gen if gen else self.self_attn.q_proj
        mlp = self.mlp_mot_gen if gen else self.mlp
        norm = self.norm_mot_gen if gen else self.norm
        h = h + attn(norm(h.float()).to(h.dtype)) * self.shared_scale[0].to(h.dtype)
        return h + mlp.up_proj(h)[..., :H]


class Model(nn.Module):
    def __init__(self, n_layers):
        super().__init__()
        self.layers = nn.ModuleList([Layer(7 * i + 1) for i in range(n_layers)])
        self.final = nn.LayerNorm(H)

    def forward(self, h, **flags):
        for layer in self.layers:
            h = layer(h, **flags)
        return self.final(h.float())


UND = {"exist_non_image_gen_tokens": True, "exist_image_gen_tokens": False}
GEN = {"exist_non_image_gen_tokens": False, "exist_image_gen_tokens": True}


@pytest.mark.parametrize("prefetch", [0, 1, 2])
def test_streamed_layers_match_resident_layers(dev, prefetch):
    print(f"case offload prefetch={prefetch}", flush=True)
    torch.manual_seed(0)
    host = Model(5).eval()
    for l in host.layers:   # shared_scale 0 would hide the attention branch
        l.shared_scale.fill_(0.5)
    resident = copy.deepcopy(host).to(dev)
    xs = [synthetic.make_activations(m, H, seed=m).to(dev) for m in (1, 9, 40)]
    want = {(m, k): resident(x, **f).clone() for m, x in zip((1, 9, 40), xs) for k, f in (("und", UND), ("gen", GEN))}
    wrapped = LayerOffloadWrapper(host, "layers", dev, prefetch_count=prefetch)
    assert host.final.weight.device.type == "cuda"                       # outside the layer list: resident
    assert host.layers[0].self_attn.q_proj.weight.device.type == "cpu"   # inside: on the host until needed
    assert host.layers[0].self_attn.q_proj.weight.is_pinned()
    assert host.layers[0].self_attn.q_proj.weight.quant_type == 8
    for _ in range(3):                                                    # repeated passes reuse the slots
        for m, x in zip((1, 9, 40), xs):
            got = wrapped(x, **UND)
            assert torch.equal(got, want[(m, "und")])
    total, by_group = wrapped.transfer_stats()
    assert by_group[GROUP_GENERATION] == 0 and by_group[GROUP_UNDERSTANDING] > 0
    ring = wrapped.store.slots_allocated()
    assert ring[GROUP_UNDERSTANDING] == 1 + prefetch and ring[GROUP_GENERATION] == 0
    before = by_group[GROUP_UNDERSTANDING]
    for m, x in zip((1, 9, 40), xs):                                      # tower change: drain, then the other tower
        assert torch.equal(wrapped(x, **GEN), want[(m, "gen")])
    total, by_group = wrapped.transfer_stats()
    assert by_group[GROUP_GENERATION] > 0
    assert by_group[GROUP_UNDERSTANDING] == before                        # and nothing of the first tower
    assert torch.equal(wrapped(xs[0], **UND), want[(1, "und")])
    # no flags: both towers and the shared tensors come in
    assert torch.equal(wrapped(xs[1]), want[(9, "und")])
    assert wrapped.store.slots_allocated()[GROUP_GENERATION] >= 1
    ring = dict(wrapped.store.slots_allocated())
    for _ in range(2):
        wrapped(xs[1])
    assert wrapped.store.slots_allocated() == ring                        # steady state: nothing new is allocated
    wrapped.teardown()
    assert all(p.device.type == "cpu" for p in host.parameters())
    assert not host.layers[0]._forward_pre_hooks and not host.layers[0]._forward_hooks


def test_generation_tower_can_stay_resident(dev):
    print("case offload keep_generation_resident", flush=True)
    host = Model(3).eval()
    resident = copy.deepcopy(host).to(dev)
    x = synthetic.make_activations(4, H, seed=3).to(dev)
    want = resident(x, **GEN)
    wrapped = LayerOffloadWrapper(host, "layers", dev, prefetch_count=1, keep_generation_resident=True)
    for _ in range(3):
        assert torch.equal(wrapped(x, **GEN), want)
    _total, by_group = wrapped.transfer_stats()
    assert by_group[GROUP_GENERATION] <= 3 * _padded(wrapped, GROUP_GENERATION)   # copied once, not once per pass
    assert all(wrapped.store.is_on_gpu(i, frozenset({GROUP_GENERATION})) for i in range(3))
    assert not wrapped.store.is_on_gpu(1, frozenset({GROUP_SHARED}))      # the shared group is still streamed
    wrapped.teardown()


def _padded(wrapped, group):
    return max(wrapped.store.group_nbytes(i, group) for i in range(wrapped.store.num_layers)) + 256 * 16


def test_stacked_qkv_copy_is_released_when_the_offloader_takes_the_weights(dev):
    """q / k / v stacked into one device tensor (what the one-call loader does by default), then wrapped for layer
    offload: the weights move into the pinned arenas, so the stack must let go of its device copy."""
    print("case offload releases the q|k|v stack", flush=True)
    from sensenova_u1_amd import GGUFLinear, GGUFParameter, stack_shared_input_projections

    def q(n, k, seed):
        lin = GGUFLinear(k, n, bias=False, compute_dtype=torch.bfloat16, device="meta")
        lin.weight = GGUFParameter(synthetic.make_packed(8, n, k, seed=seed, device=dev), quant_type=8)
        return lin

    class Attn(nn.Module):
        def __init__(self, s):
            super().__init__()
            self.q_proj, self.k_proj, self.v_proj = q(512, 512, s), q(128, 512, s + 1), q(128, 512, s + 2)

        def forward(self, h):
            return self.q_proj(h) + torch.cat([self.k_proj(h), self.v_proj(h)] * 2, dim=-1)

    class M(nn.Module):
        def __init__(self):
            super().__init__()
            self.layers = nn.ModuleList([Attn(10 * i) for i in range(3)])

        def forward(self, h):
            for l in self.layers:
                h = l(h)
            return h

    model = M().eval()
    x = synthetic.make_activations(1, 512, seed=3, device=dev)
    want = model(x)
    assert stack_shared_input_projections(model) == 3
    stacks = [l.q_proj.__dict__["_shared_stack"] for l in model.layers]
    assert torch.equal(model(x), want) and all(s.intact() for s in stacks)
    wrapped = LayerOffloadWrapper(model, "layers", dev, prefetch_count=1)
    assert all(s.stacked is None for s in stacks)
    assert not any("_shared_stack" in m.__dict__ for l in model.layers for m in (l.q_proj, l.k_proj, l.v_proj))
    assert torch.equal(wrapped(x), want)
    wrapped.teardown()
