"""GPU: the decode MLP as one entry point (``sngguf_mlp_decode``): one launch at the 8B model's shape for up to two rows
in Q8_0 and in the K-quant mixes (Q4_K gate / up with a Q6_K or Q4_K down projection), the separate launches everywhere
else.  Against the separate launches of the library (the gated activations come out of the same arithmetic in the same
order, so only the down projection's order of summation differs - and, for the K-quants with the norm folded in, the
order in which the sum of squares is added) and against the CPU oracle on sampled output columns; consecutive calls,
graph replays (the hand-over state advances by itself), the bounded wait."""
import pytest
import torch

from oracle import gguf_oracle as go
from sensenova_u1_amd import ops, synthetic

pytestmark = pytest.mark.gpu
TOL = 1e-3
H, I = 4096, 12288
EPS = 1e-6


def _weights(dev, qt_gu=go.Q8_0, qt_d=go.Q8_0, seed=0, hidden=H, inter=I):
    return (synthetic.make_packed(qt_gu, inter, hidden, seed=seed + 1, device=dev),
            synthetic.make_packed(qt_gu, inter, hidden, seed=seed + 2, device=dev),
            synthetic.make_packed(qt_d, hidden, inter, seed=seed + 3, device=dev))


def _activations_left_in(ws, m, inter=I):
    """The gated activations of the last one-launch call: 8-byte words {two bf16, tag} from byte 8192 on."""
    words = ws[8192:8192 + 4 * m * inter].view(torch.int32).view(m, inter // 2, 2)
    return words[:, :, 0].contiguous().view(torch.bfloat16).view(m, inter)


def _separate(x, gamma, gate, up, down, qt_gu, qt_d, residual, num):
    m = x.shape[0]
    h = torch.empty((m, gate.shape[0]), dtype=torch.bfloat16, device=x.device)
    if gamma is not None and ops.rmsnorm_fits(qt_gu, m, x.shape[1]):
        ops.rmsnorm_gate_up_silu_into(x, gamma, EPS, gate, up, qt_gu, h, num)
    else:
        xn = ops.rms_norm(x, gamma, EPS) if gamma is not None else x
        ops.gate_up_silu_into(xn, gate, up, qt_gu, h, num)
    y = torch.empty((m, down.shape[0]), dtype=torch.bfloat16, device=x.device)
    if residual is not None:
        ops.linear_residual_into(h, down, qt_d, None, residual, y, num)
    else:
        ops.linear_into(h, down, qt_d, None, y, num)
    return y, h


ONE_LAUNCH_TYPES = [(go.Q8_0, go.Q8_0), (go.Q4_K, go.Q6_K), (go.Q4_K, go.Q4_K)]


@pytest.mark.parametrize("m", [1, 2])
@pytest.mark.parametrize("num", [ops.NUM_GGML_FP32, ops.NUM_UPSTREAM_FP16])
@pytest.mark.parametrize("qt_gu,qt_d", ONE_LAUNCH_TYPES)
def test_one_launch_mlp_matches_the_separate_launches_and_the_oracle(dev, c_oracle, m, num, qt_gu, qt_d):
    print(f"case mlp_decode {qt_gu}/{qt_d} m={m} num={num}", flush=True)
    assert ops.mlp_decode_fits(qt_gu, qt_d, m, H, I)
    gate, up, down = _weights(dev, qt_gu, qt_d, seed=10 * m)
    ws = torch.zeros(ops.mlp_decode_workspace_bytes(m, H, I), dtype=torch.uint8, device=dev)
    gen = torch.Generator().manual_seed(m)
    gamma = (torch.rand(H, generator=gen) * 1.5 + 0.25).to(torch.bfloat16).to(dev)
    for use_gamma in (False, True):
        for use_res in (False, True):
            x = synthetic.make_activations(m, H, seed=100 + m + 2 * use_gamma + use_res, device=dev)
            res = synthetic.make_activations(m, H, seed=200 + m, device=dev) if use_res else None
            g = gamma if use_gamma else None
            y = torch.full((m, H), float("nan"), dtype=torch.bfloat16, device=dev)
            ops.mlp_decode_into(x, g, EPS, gate, up, qt_gu, down, qt_d, res, y, ws, num)
            want, h_sep = _separate(x, g, gate, up, down, qt_gu, qt_d, res, num)
            assert bool(torch.isfinite(y.float()).all())
            # the gated activations the launch left in the workspace are the pair kernel's own (K-quants with the norm
            # folded in: the workgroup adds the sum of squares over twelve wavefronts where the pair's launch adds it
            # over two, so 1 / rms may differ in its last bits and a normalized value that sat on a bf16 tie with it)
            h_ws = _activations_left_in(ws, m)
            if qt_gu == go.Q8_0 or not use_gamma:
                assert torch.equal(h_ws, h_sep), (use_gamma, use_res)
                assert go.rel_l2(y.cpu(), want.cpu()) <= 1e-4, (use_gamma, use_res)
            else:
                assert go.rel_l2(h_ws.cpu(), h_sep.cpu()) <= 3e-4, (use_gamma, use_res)
                assert go.rel_l2(y.cpu(), want.cpu()) <= 5e-4, (use_gamma, use_res)
            assert not ops.mlp_decode_gave_up(ws)
            # the oracle, stage by stage (the tolerance is stated per linear): the gated activations on sampled columns
            # against oracle norm + gate / up / SiLU, and sampled outputs against the oracle's down projection of the
            # activations the launch itself produced
            cols = torch.randint(0, H, (40,), generator=gen)
            icols = torch.randint(0, I, (64,), generator=gen)
            xn = go.qwen3_rms_norm(x.cpu(), gamma.cpu(), EPS) if use_gamma else x.cpu()
            hg = c_oracle.silu_mul(go.gguf_linear_forward(xn, gate[icols.to(dev)].cpu(), qt_gu, None, numerics=num),
                                   go.gguf_linear_forward(xn, up[icols.to(dev)].cpu(), qt_gu, None, numerics=num))
            assert go.rel_l2(h_ws[:, icols.to(dev)].cpu(), hg) <= TOL, (use_gamma, use_res)
            yo = go.gguf_linear_forward(h_ws.cpu(), down[cols.to(dev)].cpu(), qt_d, None, numerics=num)
            if use_res:
                yo = (res.cpu()[:, cols].float() + yo.float()).to(torch.bfloat16)
            assert go.rel_l2(y[:, cols.to(dev)].cpu(), yo) <= TOL, (use_gamma, use_res)


@pytest.mark.parametrize("qt_gu,qt_d", ONE_LAUNCH_TYPES[:2])
def test_consecutive_calls_and_graph_replays_advance_the_hand_over_state(dev, qt_gu, qt_d):
    print(f"case mlp_decode replays {qt_gu}/{qt_d}", flush=True)
    m = 1
    sets = [_weights(dev, qt_gu, qt_d, seed=50 + 10 * i) for i in range(3)]
    ws = torch.zeros(ops.mlp_decode_workspace_bytes(m, H, I), dtype=torch.uint8, device=dev)
    x = synthetic.make_activations(m, H, seed=7, device=dev)
    ys = [torch.empty((m, H), dtype=torch.bfloat16, device=dev) for _ in sets]
    wants = [_separate(x, None, *w, qt_gu, qt_d, None, 1)[0] for w in sets]

    def run():
        for w, y in zip(sets, ys):
            ops.mlp_decode_into(x, None, EPS, *w[:2], qt_gu, w[2], qt_d, None, y, ws, 1)

    for _ in range(3):
        run()
    torch.cuda.synchronize()
    for y, w in zip(ys, wants):
        assert go.rel_l2(y.cpu(), w.cpu()) <= 1e-4
    first = [y.clone() for y in ys]
    gen_word = lambda: int(ws[0:4].view(torch.int32).item())
    assert gen_word() == 9
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    for rep in range(4):
        for y in ys:
            y.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for y, f in zip(ys, first):
            assert torch.equal(y, f), rep
        ops.linear(x, sets[0][0], qt_gu)            # eager work between the replays
        torch.cuda.synchronize()
    assert gen_word() == 9 + 3 * 4 and not ops.mlp_decode_gave_up(ws)


@pytest.mark.parametrize("qt_gu,qt_d", ONE_LAUNCH_TYPES[:2])
def test_a_bounded_wait_that_gives_up_still_ends_the_launch(dev, qt_gu, qt_d):
    """spin_limit < 0: a workgroup that does not find every flag set at its first poll gives up at once, says so in the
    status word and finishes; the state still advances and a following ordinary call on the workspace is right."""
    print(f"case mlp_decode give-up {qt_gu}/{qt_d}", flush=True)
    m = 1
    gate, up, down = _weights(dev, qt_gu, qt_d, seed=90)
    ws = torch.zeros(ops.mlp_decode_workspace_bytes(m, H, I), dtype=torch.uint8, device=dev)
    x = synthetic.make_activations(m, H, seed=8, device=dev)
    y = torch.empty((m, H), dtype=torch.bfloat16, device=dev)
    ops.mlp_decode_into(x, None, EPS, gate, up, qt_gu, down, qt_d, None, y, ws, 1, spin_limit=-1)
    torch.cuda.synchronize()
    assert int(ws[0:4].view(torch.int32).item()) == 1          # generation advanced: every workgroup came through
    gave_up = ops.mlp_decode_gave_up(ws)
    print(f"  gave up: {gave_up}", flush=True)
    off = int(ops.load_library().sngguf_mlp_decode_status_offset())
    ws[off:off + 4].zero_()
    ops.mlp_decode_into(x, None, EPS, gate, up, qt_gu, down, qt_d, None, y, ws, 1)
    want = _separate(x, None, gate, up, down, qt_gu, qt_d, None, 1)[0]
    assert go.rel_l2(y.cpu(), want.cpu()) <= 1e-4 and not ops.mlp_decode_gave_up(ws)


@pytest.mark.parametrize("qt_gu,qt_d,m,hidden,inter", [(go.Q8_0, go.Q8_0, 3, H, I), (go.Q8_0, go.Q8_0, 16, H, I), (go.Q4_K, go.Q6_K, 3, H, I),
                                                        (go.Q6_K, go.Q6_K, 1, H, I), (go.Q8_0, go.Q6_K, 1, H, I), (go.Q4_K, go.Q8_0, 2, H, I),
                                                        (go.Q8_0, go.Q8_0, 2, 2048, 6144), (go.Q4_K, go.Q4_K, 3, 1024, 2816),
                                                        (go.Q8_0, go.Q8_0, 1, 512, 1536)])
def test_other_shapes_and_types_run_the_separate_launches(dev, qt_gu, qt_d, m, hidden, inter):
    print(f"case mlp_decode fallback {qt_gu}/{qt_d} m={m} {hidden}/{inter}", flush=True)
    assert not ops.mlp_decode_fits(qt_gu, qt_d, m, hidden, inter)
    gate, up, down = _weights(dev, qt_gu, qt_d, seed=3, hidden=hidden, inter=inter)
    ws = torch.zeros(ops.mlp_decode_workspace_bytes(m, hidden, inter), dtype=torch.uint8, device=dev)
    x = synthetic.make_activations(m, hidden, seed=9, device=dev)
    gamma = (torch.rand(hidden, generator=torch.Generator().manual_seed(4)) + 0.5).to(torch.bfloat16).to(dev)
    res = synthetic.make_activations(m, hidden, seed=10, device=dev)
    for g in (None, gamma):
        for r in (None, res):
            y = torch.full((m, hidden), float("nan"), dtype=torch.bfloat16, device=dev)
            ops.mlp_decode_into(x, g, EPS, gate, up, qt_gu, down, qt_d, r, y, ws, 1)
            assert torch.equal(y, _separate(x, g, gate, up, down, qt_gu, qt_d, r, 1)[0])


def test_argument_errors(dev):
    gate, up, down = _weights(dev, seed=1, hidden=512, inter=1536)
    x = synthetic.make_activations(1, 512, seed=1, device=dev)
    y = torch.empty((1, 512), dtype=torch.bfloat16, device=dev)
    small = torch.zeros(1024, dtype=torch.uint8, device=dev)
    with pytest.raises(ops.SnGgufError):
        ops.mlp_decode_into(x, None, EPS, gate, up, go.Q8_0, down, go.Q8_0, None, y, small, 1)
    assert ops.mlp_decode_workspace_bytes(17, 512, 1536) == 0


def test_gated_mlp_takes_the_one_launch_route_and_can_be_told_not_to(dev, monkeypatch):
    """modality.gated_mlp (what load_gguf_model points Qwen3MLP-shaped modules at): one or two rows of the model's shape
    go through sngguf_mlp_decode, with the norm and the residual add inside; switched off, the separate launches give
    the same values up to the order of the down projection's partial sums."""
    print("case mlp_decode through gated_mlp", flush=True)
    from sensenova_u1_amd import GGUFLinear, GGUFParameter, modality

    def lin(packed, n, k):
        m = GGUFLinear(k, n, bias=False, compute_dtype=torch.bfloat16, device="meta")
        m.weight = GGUFParameter(packed, quant_type=go.Q8_0)
        return m

    gate, up, down = _weights(dev, seed=70)
    g, u, d = lin(gate, I, H), lin(up, I, H), lin(down, H, I)
    gamma = (torch.rand(H, generator=torch.Generator().manual_seed(5)) + 0.5).to(torch.bfloat16).to(dev)
    calls = []
    real = ops.mlp_decode_into
    monkeypatch.setattr(ops, "mlp_decode_into", lambda *a, **k: (calls.append(a[0].shape[0]), real(*a, **k))[1])
    for m in (1, 3, 5):
        x = synthetic.make_activations(m, H, seed=m, device=dev).reshape(1, m, H)
        res = synthetic.make_activations(m, H, seed=10 + m, device=dev).reshape(1, m, H)
        for gm, rs in ((None, None), (gamma, res)):
            calls.clear()
            got = modality.gated_mlp(x, g, u, d, gm, EPS, rs)
            assert got.shape == (1, m, H) and len(calls) == (1 if m <= 2 else 0)
            monkeypatch.setattr(modality, "ONE_LAUNCH_MLP", False)
            want = modality.gated_mlp(x, g, u, d, gm, EPS, rs)
            monkeypatch.setattr(modality, "ONE_LAUNCH_MLP", True)
            assert go.rel_l2(got.cpu(), want.cpu()) <= 1e-4
            if m > 2:
                assert torch.equal(got, want)
    assert not ops.mlp_decode_gave_up(ops.mlp_decode_workspace(dev, 1, H, I))
