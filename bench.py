#!/usr/bin/env python3
"""Benchmark of the GGUF quantized-linear hot path on one MI355X.

Headline leg (``value``): the Q8_0 SiLU-gated MLP of one decoder layer at decode, M = 1
(gate / up 4096 -> 12288, down 12288 -> 4096).  One *step* is one pass of that MLP over one
layer's packed weights; consecutive steps walk over ``--layers`` distinct weight sets (default
16 x 160 MB = 2.6 GB, far beyond the 256 MB last-level cache), so every step streams its
weights from HBM.  ``value`` is algorithmic bytes per step / wall time per step.

Further legs in the same JSON line: the same MLP at M = 4 and 16, and the M = 4096 Q8_0
generation-tower projections (q, k, v, o, gate, up, down of one tower-layer) on the MFMA GEMM,
reported in TFLOP/s.  ``roofline`` belongs to the dominant kernel of the headline leg (the fused
gate/up GEMV), timed alone with HIP events; ``gemm.roofline`` to the largest GEMM (gate shape).
``cpu_baseline`` times the CPU oracle's port of the reference forward on the host cores.

All inputs are synthetic, seeded, resident in HBM before the timed region starts.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HIDDEN, INTER, KV = 4096, 12288, 1024
# HBM bytes per launch of the dominant kernels: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per dispatch,
# each scaled by what the same counter reads for the plain 256 MiB elementwise copy that
# --calibrate-copy runs in the same process; None = not measured for this build.
MEASURED_TRAFFIC = {"mlp_one_launch_m1": 164774013, "gemv_gate_up_m1": 107629683, "gemm_gate_m4096": 516359845, "gemm_dense_gate_m4096": 705462160}
HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
Q8_0, Q4_K, Q6_K = 8, 12, 14
BLOCK = {Q8_0: (32, 34), Q4_K: (256, 144), Q6_K: (256, 210)}   # elements, bytes per block


def packed_bytes(qt: int, n: int, k: int) -> int:
    bs, ts = BLOCK[qt]
    return n * (k // bs) * ts


def linear_bytes(m: int, n: int, k: int, qt: int = Q8_0) -> int:
    """Algorithmic bytes of one quantized linear: packed weight once, bf16 x once, bf16 y once."""
    return packed_bytes(qt, n, k) + 2 * m * k + 2 * m * n


def mlp_bytes(m: int, gate_up_type: int = Q8_0, down_type: int = Q8_0) -> int:
    return 2 * linear_bytes(m, INTER, HIDDEN, gate_up_type) + linear_bytes(m, HIDDEN, INTER, down_type)


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=512)
    ap.add_argument("--warmup", type=int, default=64)
    ap.add_argument("--layers", type=int, default=16, help="distinct MLP weight sets the steps rotate over")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-gemm", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the K-quant (configs[3]) and grouped (configs[4]) legs")
    ap.add_argument("--gemm-steps", type=int, default=20)
    ap.add_argument("--gemm-warmup", type=int, default=10,
                    help="untimed tower-layer passes before the GEMM leg (about 20 ms: the shader clock settles "
                         "under the matrix-core load within that time)")
    ap.add_argument("--settle-ms", type=float, default=20.0,
                    help="untimed repetitions of each leg's own timed work (the captured graph) for at least this long "
                         "before its timed region, so that a short region (--steps 20) is measured in the steady state of a "
                         "decode loop (clocks, translation caches, graph upload) like a long one")
    ap.add_argument("--numerics", type=int, default=1, help="1 = upstream fp16 chain (drop-in), 0 = ggml fp32")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run plain 256 MiB elementwise device copies (a known-size reference for scaling the "
                         "FETCH_SIZE / WRITE_SIZE hardware counters when profiling with rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus N with N > 1 is not supported "
              "(the path would shard by output rows; no multi-GPU code is part of it)", file=sys.stderr)
        sys.exit(2)

    import torch

    from sensenova_u1_amd import ops, synthetic

    if not torch.cuda.is_available():
        print("bench.py: no HIP device", file=sys.stderr)
        sys.exit(1)
    ops.load_library()
    dev = torch.device("cuda:0")
    num = args.numerics
    K, W, L = args.steps, args.warmup, args.layers

    if args.calibrate_copy:
        src = torch.randint(0, 255, (256 * 1024 * 1024,), dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(4):
            torch.bitwise_not(src, out=dst)  # one elementwise kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    # ---- synthetic weights, resident in HBM --------------------------------------------------
    layers = []
    for i in range(L):
        layers.append((synthetic.make_packed(Q8_0, INTER, HIDDEN, seed=1000 + 3 * i, device=dev),
                       synthetic.make_packed(Q8_0, INTER, HIDDEN, seed=1001 + 3 * i, device=dev),
                       synthetic.make_packed(Q8_0, HIDDEN, INTER, seed=1002 + 3 * i, device=dev)))
    torch.cuda.synchronize()

    settle_replays = []

    def run_region(fn, n_steps: int, warmup: int, settle_ms: float = None):
        """W warm-up steps, then exactly n_steps steps timed (wall clock around a synchronised
        region, and HIP events on the launch stream).  Returns (wall_ms, event_ms).

        Between the warm-up and the timed region the SAME work (the captured graph, or the eager loop)
        is repeated untimed until ``settle_ms`` of wall time have passed: a region of 20 steps lasts
        under a millisecond, in which neither the shader and memory clocks nor the translation caches
        have reached the state every later step of a decode loop runs in.  The timed region is still
        exactly n_steps steps; the figure is then the same whatever --steps is."""
        settle = args.settle_ms if settle_ms is None else settle_ms
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        graph = None
        if not args.no_graph:
            try:
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    for i in range(n_steps):
                        fn(warmup + i)
            except Exception as exc:  # capture unsupported: time eager launches instead
                print(f"bench.py: graph capture failed ({exc}); timing eager launches", file=sys.stderr)
                graph = None
                torch.cuda.synchronize()

        def once():
            if graph is not None:
                graph.replay()
            else:
                for i in range(n_steps):
                    fn(warmup + i)

        # the first launch of an instantiated graph also uploads it to the device (4 - 8 % on top of a 512-node graph of
        # 24 us kernels, measured); torch exposes no hipGraphUpload, so the untimed replays do it
        t_settle = time.perf_counter()
        reps = 0
        while reps < 1 or (time.perf_counter() - t_settle) * 1e3 < settle:
            once()
            reps += 1
            if reps % 8 == 0:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        settle_replays.append(reps)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        once()
        e1.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        return (t1 - t0) * 1e3, e0.elapsed_time(e1)

    def mlp_leg(m: int, n_steps: int, warmup: int, layers=layers, gate_up_type: int = Q8_0, down_type: int = Q8_0):
        """The MLP step as two launches (fused gate/up + SiLU, then down), and each of the two alone."""
        x = synthetic.make_activations(m, HIDDEN, seed=7, device=dev)
        h = torch.empty((m, INTER), dtype=torch.bfloat16, device=dev)
        y = torch.empty((m, HIDDEN), dtype=torch.bfloat16, device=dev)
        nl = len(layers)

        def step(i):
            gate, up, down = layers[i % nl]
            ops.gate_up_silu_into(x, gate, up, gate_up_type, h, num)
            ops.linear_into(h, down, down_type, None, y, num)

        def gate_up_only(i):
            gate, up, _ = layers[i % nl]
            ops.gate_up_silu_into(x, gate, up, gate_up_type, h, num)

        def down_only(i):
            ops.linear_into(h, layers[i % nl][2], down_type, None, y, num)

        wall, ev = run_region(step, n_steps, warmup)
        _, ev_gu = run_region(gate_up_only, n_steps, warmup)
        _, ev_dn = run_region(down_only, n_steps, warmup)
        return wall, ev, ev_gu / n_steps, ev_dn / n_steps

    def mlp_one_launch_leg(m: int, n_steps: int, warmup: int, lay=None, qt_gu=Q8_0, qt_down=Q8_0):
        """The MLP step as modality.gated_mlp runs it by default for one or two rows: sngguf_mlp_decode, ONE launch."""
        lay = layers if lay is None else lay
        x = synthetic.make_activations(m, HIDDEN, seed=7, device=dev)
        y = torch.empty((m, HIDDEN), dtype=torch.bfloat16, device=dev)
        ws = torch.zeros(ops.mlp_decode_workspace_bytes(m, HIDDEN, INTER), dtype=torch.uint8, device=dev)
        nl = len(lay)

        def step(i):
            gate, up, down = lay[i % nl]
            ops.mlp_decode_into(x, None, 1e-6, gate, up, qt_gu, down, qt_down, None, y, ws, num)

        wall, ev = run_region(step, n_steps, warmup)
        torch.cuda.synchronize()
        if ops.mlp_decode_gave_up(ws):
            raise RuntimeError("bench.py: a one-launch MLP gave up waiting for its workgroups; the figure would be void")
        return wall, ev

    one_launch = ops.mlp_decode_fits(Q8_0, Q8_0, 1, HIDDEN, INTER)
    wall2, ev2, gu_ms, dn_ms = mlp_leg(1, K, W)
    step_bytes = mlp_bytes(1)
    if one_launch:
        wall1, ev1 = mlp_one_launch_leg(1, K, W)
    else:
        wall1, ev1 = wall2, ev2
    ms_per_step = wall1 / K
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    gu_bytes = 2 * linear_bytes(1, INTER, HIDDEN)
    gu_gbps = gu_bytes / (gu_ms * 1e-3) / 1e9
    dn_bytes = linear_bytes(1, HIDDEN, INTER)
    dev_gbps = step_bytes / (ev1 / K * 1e-3) / 1e9
    two_gbps = step_bytes / (wall2 / K * 1e-3) / 1e9

    if one_launch:
        roofline = {
            "kernel": "sngguf::mlp_q8_decode_kernel<upstream_fp16> (gate/up + SiLU + down of the M=1 MLP in one launch: the whole step)",
            "bound": "hbm",
            "achieved": round(dev_gbps, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(dev_gbps / HBM_PEAK_GBPS, 4),
            "traffic": MEASURED_TRAFFIC["mlp_one_launch_m1"],
            "bytes_per_launch": step_bytes,
            "avg_launch_us": round(ev1 / K * 1e3, 3),
            "device_ms_per_step": round(ev1 / K, 6),
            "timing": "HIP events on the launch stream around the timed replay of the graph of `steps` launches",
        }
    else:
        roofline = {
            "kernel": "sngguf::gemv_q8_span_kernel<upstream_fp16, gated> (fused gate/up + SiLU, M=1)",
            "bound": "hbm",
            "achieved": round(gu_gbps, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(gu_gbps / HBM_PEAK_GBPS, 4),
            "traffic": MEASURED_TRAFFIC["gemv_gate_up_m1"],
            "bytes_per_launch": gu_bytes,
            "avg_launch_us": round(gu_ms * 1e3, 3),
            "device_ms_per_step": round(ev1 / K, 6),
            "timing": "HIP events on the launch stream around the timed replay of a graph of `steps` gate/up launches",
        }

    result = {
        "metric": "Q8_0 dequant-GEMV HBM GB/s (% of peak); M=4096 dequant-GEMM TFLOP/s",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "configs[1]: Q8_0 MLP of one decoder layer, text decode M=1 "
                        "(gate/up 4096->12288 with SiLU, down 12288->4096)",
            "route": ("sngguf_mlp_decode: the whole MLP in one launch (what modality.gated_mlp runs by default for one or two rows)"
                      if one_launch else "sngguf_gate_up_silu + sngguf_linear: two launches"),
            "layers_rotated": L,
            "bytes_per_step": step_bytes,
            "graph": not args.no_graph,
            "settle_ms": args.settle_ms,
            "untimed_replays_before_timed_region": settle_replays[0],
            "numerics": "upstream_fp16" if num == 1 else "ggml_fp32",
        },
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "device_ms_per_step": round(ev1 / K, 6),
        "roofline": roofline,
        "two_launches": {
            "what": "the same step as sngguf_gate_up_silu + sngguf_linear (modality.ONE_LAUNCH_MLP = False, and every row count "
                    "beyond two): the fused gate/up + SiLU kernel, then the down projection",
            "value": round(two_gbps, 1), "unit": "GB/s", "pct_of_hbm_peak": round(100.0 * two_gbps / HBM_PEAK_GBPS, 2),
            "ms_per_step": round(wall2 / K, 6), "device_ms_per_step": round(ev2 / K, 6),
            "gate_up": {
                "kernel": "sngguf::gemv_q8_span_kernel<upstream_fp16, gated> (fused gate/up + SiLU, M=1)",
                "achieved": round(gu_gbps, 1), "unit": "GB/s", "frac": round(gu_gbps / HBM_PEAK_GBPS, 4),
                "traffic": MEASURED_TRAFFIC["gemv_gate_up_m1"], "bytes_per_launch": gu_bytes, "avg_launch_us": round(gu_ms * 1e3, 3),
            },
            "down_proj": {
                "kernel": "sngguf::gemv_q8_mfma_kernel<upstream_fp16> (down 12288->4096, M=1)",
                "achieved": round(dn_bytes / (dn_ms * 1e-3) / 1e9, 1), "unit": "GB/s", "frac": round(dn_bytes / (dn_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                "bytes_per_launch": dn_bytes, "avg_launch_us": round(dn_ms * 1e3, 3),
            },
        },
    }

    # ---- what the memory system gives a launch that only reads: the library's streaming-read probe over a buffer
    # ten times the last-level cache, as one launch over all of it and as launches of the gate/up kernel's size ------
    if not args.no_extra:
        import ctypes
        lib = ops.load_library()
        chunk = (gu_bytes + 4095) // 4096 * 4096
        n_chunks = 24
        probe_buf = torch.empty(n_chunks * chunk, dtype=torch.uint8, device=dev)
        probe_buf.view(torch.int64).random_()
        probe_out = torch.empty(int(lib.sngguf_probe_stream_read_out_bytes()), dtype=torch.uint8, device=dev)
        torch.cuda.synchronize()

        def probe(off, nbytes, nt, wgs=0):
            rc = lib.sngguf_probe_stream_read(ctypes.c_void_p(probe_buf.data_ptr() + off), nbytes, ctypes.c_void_p(probe_out.data_ptr()),
                                              wgs, nt, ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
            assert rc == 0, rc

        pr = {}
        for nt in (1, 0):
            _, ev_all = run_region(lambda i: probe(0, n_chunks * chunk, nt), 8, 2)
            _, ev_chunk = run_region(lambda i: probe((i % n_chunks) * chunk, chunk, nt), max(K, 48), 8)
            _, ev_chunk256 = run_region(lambda i: probe((i % n_chunks) * chunk, chunk, nt, 256), max(K, 48), 8)
            tag = "nontemporal" if nt else "plain"
            pr[tag] = {"one_launch_over_all_GBps": round(n_chunks * chunk / (ev_all / 8 * 1e-3) / 1e9, 1),
                       "launches_of_gate_up_size_GBps": round(chunk / (ev_chunk / max(K, 48) * 1e-3) / 1e9, 1),
                       "launches_of_gate_up_size_us": round(ev_chunk / max(K, 48) * 1e3, 3),
                       "launches_of_gate_up_size_256_workgroups_us": round(ev_chunk256 / max(K, 48) * 1e3, 3)}
        best = max(v["one_launch_over_all_GBps"] for v in pr.values())
        best_chunk = max(v["launches_of_gate_up_size_GBps"] for v in pr.values())
        result["hbm_read_probe"] = {
            "what": "sngguf_probe_stream_read: a kernel that only reads (16 bytes per lane and request, eight in flight, one "
                    "word per workgroup written), over a 2.6 GB buffer: one launch over all of it, and back-to-back launches "
                    "of the gate/up kernel's 107 MB each on distinct ranges (graph replay, HIP events)",
            "buffer_bytes": n_chunks * chunk, "bytes_per_sized_launch": chunk, **pr,
            "achievable_hbm_read_GBps": best, "achievable_frac_of_peak": round(best / HBM_PEAK_GBPS, 4),
            "achievable_at_gate_up_launch_size_GBps": best_chunk,
        }
        result["roofline"]["achievable_hbm_read_GBps"] = best
        result["roofline"]["frac_of_achievable"] = round(result["roofline"]["achieved"] / best, 4)
        result["two_launches"]["gate_up"]["achievable_at_this_launch_size_GBps"] = best_chunk
        result["two_launches"]["gate_up"]["frac_of_achievable_at_this_launch_size"] = round(gu_gbps / best_chunk, 4)
        del probe_buf, probe_out

    # ---- same MLP at M = 4 and 16 --------------------------------------------------------------
    decode = {}
    for m in (4, 16):
        k2 = max(64, K // 4)
        wall, ev, gu, dn = mlp_leg(m, k2, min(W, 16))
        gbps = mlp_bytes(m) / (wall / k2 * 1e-3) / 1e9
        decode[f"M{m}"] = {"value": round(gbps, 1), "unit": "GB/s", "pct_of_hbm_peak": round(100 * gbps / HBM_PEAK_GBPS, 2),
                           "ms_per_step": round(wall / k2, 6), "gate_up_us": round(gu * 1e3, 3),
                           "down_us": round(dn * 1e3, 3)}
    result["decode_other_M"] = decode

    # ---- configs[0]: a single Q8_0 linear 4096 -> 4096 at M = 1, over 32 distinct weights (570 MB, beyond the last-level cache)
    if not args.no_extra:
        singles = [synthetic.make_packed(Q8_0, HIDDEN, HIDDEN, seed=400 + i, device=dev) for i in range(32)]
        xs1 = synthetic.make_activations(1, HIDDEN, seed=8, device=dev)
        ys1 = torch.empty((1, HIDDEN), dtype=torch.bfloat16, device=dev)
        wall_s, ev_s = run_region(lambda i: ops.linear_into(xs1, singles[i % 32], Q8_0, None, ys1, num), K, W)
        sb = linear_bytes(1, HIDDEN, HIDDEN)
        result["single_linear"] = {
            "workload": "configs[0]: one Q8_0 linear 4096 -> 4096 at M=1 (sngguf_linear), 32 distinct weights in rotation",
            "bytes_per_launch": sb, "avg_launch_us": round(ev_s / K * 1e3, 3),
            "value": round(sb / (wall_s / K * 1e-3) / 1e9, 1), "unit": "GB/s",
            "pct_of_hbm_peak": round(100 * sb / (wall_s / K * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2)}
        del singles

    # ---- the drop-in route of an unmodified Qwen3MLP.forward (modeling_qwen3.py:214-216): three GGUFLinear modules and
    # torch's SiLU and product, i.e. down_proj(act_fn(gate_proj(x)) * up_proj(x)) through Module.forward ---------------
    if not args.no_extra:
        from sensenova_u1_amd import GGUFLinear, GGUFParameter

        def as_module(packed, n, k):
            lin = GGUFLinear(k, n, bias=False, compute_dtype=torch.bfloat16, device="meta")
            lin.weight = GGUFParameter(packed, quant_type=Q8_0)
            lin.numerics = num
            return lin

        mods = [(as_module(g, INTER, HIDDEN), as_module(u, INTER, HIDDEN), as_module(d, HIDDEN, INTER)) for g, u, d in layers]
        drop = {}
        for m in (1, 4, 16):
            xm = synthetic.make_activations(m, HIDDEN, seed=7, device=dev)

            def unfused_step(i):
                gate_proj, up_proj, down_proj = mods[i % L]
                return down_proj(torch.nn.functional.silu(gate_proj(xm)) * up_proj(xm))

            kd = K if m == 1 else max(64, K // 4)
            wall_d, _ = run_region(unfused_step, kd, min(W, 16))
            gb = mlp_bytes(m) / (wall_d / kd * 1e-3) / 1e9
            drop[f"M{m}"] = {"value": round(gb, 1), "unit": "GB/s", "pct_of_hbm_peak": round(100 * gb / HBM_PEAK_GBPS, 2),
                             "ms_per_step": round(wall_d / kd, 6)}
        drop["workload"] = ("the headline MLP as an unmodified Qwen3MLP.forward runs it after the module swap: three "
                            "GGUFLinear.forward calls (gate, up, down: three decode launches), torch SiLU and product "
                            "(two elementwise launches); same algorithmic bytes as the headline step")
        result["mlp_unfused_dropin"] = drop

        # the same modules inside a Qwen3MLP-shaped nn.Module whose forward the one-call loader has pointed at the fused
        # gated MLP (modality.fuse_gated_mlps): Module.__call__ -> gated_mlp -> sngguf_gate_up_silu + sngguf_linear
        from sensenova_u1_amd import fuse_gated_mlps

        class GatedMLP(torch.nn.Module):
            def __init__(self, g, u, d):
                super().__init__()
                self.gate_proj, self.up_proj, self.down_proj, self.act_fn = g, u, d, torch.nn.SiLU()

            def forward(self, x):
                return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))

        mlps = [GatedMLP(*t) for t in mods]
        n_fused = sum(fuse_gated_mlps(mm) for mm in mlps)
        fusedleg = {}
        for m in (1, 4, 16):
            xm = synthetic.make_activations(m, HIDDEN, seed=7, device=dev)
            kd = K if m == 1 else max(64, K // 4)
            wall_f, _ = run_region(lambda i: mlps[i % L](xm), kd, min(W, 16))
            gb = mlp_bytes(m) / (wall_f / kd * 1e-3) / 1e9
            fusedleg[f"M{m}"] = {"value": round(gb, 1), "unit": "GB/s", "pct_of_hbm_peak": round(100 * gb / HBM_PEAK_GBPS, 2),
                                 "ms_per_step": round(wall_f / kd, 6)}
        fusedleg["workload"] = (f"the headline MLP through Module.forward of {n_fused} Qwen3MLP-shaped modules as "
                                "load_gguf_model leaves them (forward pointed at the fused gated MLP; output tensors "
                                "allocated per call by torch's caching allocator)")
        result["mlp_loader_fused_module"] = fusedleg
        del mods, mlps

    # ---- the same MLP on the opt-in operand-order ("tiled") copy of the weights (made once at load time) ------------
    if not args.no_extra:
        tiled = [tuple(ops.q8_0_tile(t) for t in layer) for layer in layers]
        torch.cuda.synchronize()
        tl = {}
        for m in (1, 4, 16):
            xt = synthetic.make_activations(m, HIDDEN, seed=7, device=dev)
            ht = torch.empty((m, INTER), dtype=torch.bfloat16, device=dev)
            yt = torch.empty((m, HIDDEN), dtype=torch.bfloat16, device=dev)

            def tstep(i):
                tg, tu, td = tiled[i % L]
                ops.gate_up_silu_tiled_into(xt, tg, tu, ht, num)
                ops.linear_tiled_into(ht, td, None, None, yt, num)

            kt = K if m == 1 else max(64, K // 4)
            wall_t, _ = run_region(tstep, kt, min(W, 16))
            _, ev_tg = run_region(lambda i: ops.gate_up_silu_tiled_into(xt, tiled[i % L][0], tiled[i % L][1], ht, num), kt, min(W, 16))
            _, ev_td = run_region(lambda i: ops.linear_tiled_into(ht, tiled[i % L][2], None, None, yt, num), kt, min(W, 16))
            gb = mlp_bytes(m) / (wall_t / kt * 1e-3) / 1e9
            tl[f"M{m}"] = {"value": round(gb, 1), "unit": "GB/s", "pct_of_hbm_peak": round(100 * gb / HBM_PEAK_GBPS, 2),
                           "ms_per_step": round(wall_t / kt, 6), "gate_up_us": round(ev_tg / kt * 1e3, 3),
                           "down_us": round(ev_td / kt * 1e3, 3)}
        tl["workload"] = ("the Q8_0 decode MLP of the headline leg with the weights in the opt-in operand-order copy "
                          "(sngguf_q8_0_tile, same 34 bytes per block; GGUFLinear.decode_layout = 'tiled'): "
                          "sngguf_gate_up_silu_tiled + sngguf_linear_tiled")
        result["mlp_tiled_layout"] = tl
        del tiled

    # ---- all seven linears of one decoder layer at M = 1: separate q / k / v launches against one launch over the
    # row-wise stacked q|k|v weight (modality.FusedProjections); gate/up fused with SiLU in both ---------------------
    if not args.no_extra:
        nl = 6
        attn = [(synthetic.make_packed(Q8_0, HIDDEN, HIDDEN, seed=9000 + 4 * i, device=dev),
                 synthetic.make_packed(Q8_0, KV, HIDDEN, seed=9001 + 4 * i, device=dev),
                 synthetic.make_packed(Q8_0, KV, HIDDEN, seed=9002 + 4 * i, device=dev),
                 synthetic.make_packed(Q8_0, HIDDEN, HIDDEN, seed=9003 + 4 * i, device=dev)) for i in range(nl)]
        qkv = [torch.cat(a[:3], dim=0) for a in attn]
        x1 = synthetic.make_activations(1, HIDDEN, seed=11, device=dev)
        yq = torch.empty((1, HIDDEN), dtype=torch.bfloat16, device=dev)
        yk = torch.empty((1, KV), dtype=torch.bfloat16, device=dev)
        yv = torch.empty((1, KV), dtype=torch.bfloat16, device=dev)
        yqkv = torch.empty((1, HIDDEN + 2 * KV), dtype=torch.bfloat16, device=dev)
        yo = torch.empty((1, HIDDEN), dtype=torch.bfloat16, device=dev)
        h1 = torch.empty((1, INTER), dtype=torch.bfloat16, device=dev)

        res = synthetic.make_activations(1, HIDDEN, seed=12, device=dev)
        hid = torch.empty((1, HIDDEN), dtype=torch.bfloat16, device=dev)

        def layer_rest(i, fused_residual):
            gate, up, down = layers[i % len(layers)]
            if fused_residual:
                ops.linear_residual_into(yq, attn[i % nl][3], Q8_0, None, res, hid, num)
                ops.gate_up_silu_into(hid, gate, up, Q8_0, h1, num)
                ops.linear_residual_into(h1, down, Q8_0, None, hid, yo, num)
            else:
                ops.linear_into(yq, attn[i % nl][3], Q8_0, None, yo, num)
                torch.add(res, yo, out=hid)
                ops.gate_up_silu_into(hid, gate, up, Q8_0, h1, num)
                ops.linear_into(h1, down, Q8_0, None, yo, num)
                torch.add(hid, yo, out=yq)

        def layer_separate(i):
            q, k, v, _ = attn[i % nl]
            ops.linear_into(x1, q, Q8_0, None, yq, num)
            ops.linear_into(x1, k, Q8_0, None, yk, num)
            ops.linear_into(x1, v, Q8_0, None, yv, num)
            layer_rest(i, False)

        def layer_stacked(i):
            ops.linear_into(x1, qkv[i % nl], Q8_0, None, yqkv, num)
            layer_rest(i, False)

        def layer_stacked_residual(i):
            ops.linear_into(x1, qkv[i % nl], Q8_0, None, yqkv, num)
            layer_rest(i, True)

        # the same layer with its two RMSNorms (input_layernorm in front of q|k|v, post_attention_layernorm in front of
        # the MLP): as one library norm launch each, and folded into the q|k|v and gate/up launches
        gammas = [(torch.rand(HIDDEN, generator=torch.Generator().manual_seed(70 + i)) + 0.5).to(torch.bfloat16).to(dev) for i in range(2)]
        eps = 1e-6

        def layer_norms_separate(i):
            n1 = torch.nn.functional.rms_norm(x1, (HIDDEN,), gammas[0], eps)
            ops.linear_into(n1, qkv[i % nl], Q8_0, None, yqkv, num)
            gate, up, down = layers[i % len(layers)]
            ops.linear_residual_into(yq, attn[i % nl][3], Q8_0, None, res, hid, num)
            n2 = torch.nn.functional.rms_norm(hid, (HIDDEN,), gammas[1], eps)
            ops.gate_up_silu_into(n2, gate, up, Q8_0, h1, num)
            ops.linear_residual_into(h1, down, Q8_0, None, hid, yo, num)

        def layer_norms_fused(i):
            ops.rmsnorm_linear_into(x1, gammas[0], eps, qkv[i % nl], Q8_0, None, yqkv, num)
            gate, up, down = layers[i % len(layers)]
            ops.linear_residual_into(yq, attn[i % nl][3], Q8_0, None, res, hid, num)
            ops.rmsnorm_gate_up_silu_into(hid, gammas[1], eps, gate, up, Q8_0, h1, num)
            ops.linear_residual_into(h1, down, Q8_0, None, hid, yo, num)

        # ... with the MLP, its norm and its residual add as ONE launch: three launches per layer
        ws_l = torch.zeros(ops.mlp_decode_workspace_bytes(1, HIDDEN, INTER), dtype=torch.uint8, device=dev)

        def layer_three_launches(i):
            ops.rmsnorm_linear_into(x1, gammas[0], eps, qkv[i % nl], Q8_0, None, yqkv, num)
            gate, up, down = layers[i % len(layers)]
            ops.linear_residual_into(yq, attn[i % nl][3], Q8_0, None, res, hid, num)
            ops.mlp_decode_into(hid, gammas[1], eps, gate, up, Q8_0, down, Q8_0, hid, yo, ws_l, num)

        # ... and on the tiled copies of all seven weights
        t_mlp = [tuple(ops.q8_0_tile(t) for t in layer) for layer in layers]
        t_qkv = [ops.q8_0_tile(w) for w in qkv]
        t_o = [ops.q8_0_tile(a[3]) for a in attn]
        torch.cuda.synchronize()

        def layer_tiled_norms_fused(i):
            ops.rmsnorm_linear_tiled_into(x1, gammas[0], eps, t_qkv[i % nl], None, yqkv, num)
            tg, tu, td = t_mlp[i % len(layers)]
            ops.linear_tiled_into(yq, t_o[i % nl], None, res, hid, num)
            ops.rmsnorm_gate_up_silu_tiled_into(hid, gammas[1], eps, tg, tu, h1, num)
            ops.linear_tiled_into(h1, td, None, hid, yo, num)

        k3 = max(64, K // 4)
        lbytes = (2 * linear_bytes(1, HIDDEN, HIDDEN) + 2 * linear_bytes(1, KV, HIDDEN) + mlp_bytes(1))
        legs = {}
        for name, fn, launches in (("separate", layer_separate, "6 linears + 2 adds"), ("stacked_qkv", layer_stacked, "4 linears + 2 adds"),
                                   ("stacked_qkv_fused_residual", layer_stacked_residual, "4 linears"),
                                   ("with_norms_separate", layer_norms_separate, "4 linears + 2 torch rms_norm"),
                                   ("with_norms_fused", layer_norms_fused, "4 linears, both RMSNorms inside the q|k|v and gate/up launches"),
                                   ("with_norms_fused_one_launch_mlp", layer_three_launches,
                                    "q|k|v with its norm, o with its residual add, and the whole MLP with norm and residual add as one launch: 3 launches"),
                                   ("tiled_with_norms_fused", layer_tiled_norms_fused,
                                    "as with_norms_fused on the operand-order (tiled) copies of the seven weights")):
            wall_l, _ = run_region(fn, k3, min(W, 16))
            legs[name] = {"launches": launches, "us_per_layer": round(wall_l / k3 * 1e3, 2),
                          "value": round(lbytes / (wall_l / k3 * 1e-3) / 1e9, 1), "unit": "GB/s"}
        # the same seven linears and two adds as nn.Modules with the reference's call pattern (q_proj(x), k_proj(x), v_proj(x),
        # residual + o_proj(.), residual + mlp(.) with Qwen3MLP's forward): as set_gguf2meta_model leaves them, and as
        # load_gguf_model leaves them (q / k / v on one stacked weight tensor, the MLP's forward pointed at the fused one)
        from sensenova_u1_amd import GGUFLinear, GGUFParameter, fuse_gated_mlps, stack_shared_input_projections

        def qlin(packed, n, k):
            lin = GGUFLinear(k, n, bias=False, compute_dtype=torch.bfloat16, device="meta")
            lin.weight = GGUFParameter(packed, quant_type=Q8_0)
            lin.numerics = num
            return lin

        class MLP(torch.nn.Module):
            def __init__(self, g, u, d):
                super().__init__()
                self.gate_proj, self.up_proj, self.down_proj = qlin(g, INTER, HIDDEN), qlin(u, INTER, HIDDEN), qlin(d, HIDDEN, INTER)
                self.act_fn = torch.nn.SiLU()

            def forward(self, x):
                return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))

        class Layer(torch.nn.Module):
            def __init__(self, a, mlp):
                super().__init__()
                self.q_proj, self.k_proj, self.v_proj = qlin(a[0], HIDDEN, HIDDEN), qlin(a[1], KV, HIDDEN), qlin(a[2], KV, HIDDEN)
                self.o_proj, self.mlp = qlin(a[3], HIDDEN, HIDDEN), MLP(*mlp)

            def forward(self, x):
                q, k, v = self.q_proj(x), self.k_proj(x), self.v_proj(x)
                h = x + self.o_proj(q)
                return h + self.mlp(h), k, v

        for leg, prepare in (("modules_swapped_only", None), ("modules_as_loaded", True)):
            mods_l = [Layer(attn[i], layers[i]) for i in range(nl)]   # (the second pass re-lays q / k / v into one tensor)
            if prepare:
                for ml in mods_l:
                    stack_shared_input_projections(ml)
                    fuse_gated_mlps(ml)
            wall_l, _ = run_region(lambda i: mods_l[i % nl](x1), k3, min(W, 16))
            legs[leg] = {"launches": "7 linears + SiLU, product, 2 adds through Module.forward" if not prepare else
                         "q|k|v in one launch (SharedInputStack), o, fused gate/up/SiLU, down, 2 adds through Module.forward",
                         "us_per_layer": round(wall_l / k3 * 1e3, 2), "value": round(lbytes / (wall_l / k3 * 1e-3) / 1e9, 1), "unit": "GB/s"}
            del mods_l
        result["decode_layer"] = {
            "workload": "the 7 Q8_0 linears of one decoder layer at M=1 (q,o 4096^2; k,v 4096->1024; gate/up fused with SiLU; "
                        "down) and its two residual adds; no attention; the with_norms legs add the layer's two RMSNorms; the "
                        "modules_* legs run the reference's call pattern through nn.Module forwards",
            "bytes_per_layer": lbytes, **legs,
        }
        del attn, qkv, t_mlp, t_qkv, t_o

    # ---- lm_head at decode: 151936 x 4096 Q8_0 (the vocabulary projection of the think loop), M = 1 ---------------
    if not args.no_extra:
        vocab = 151936
        heads = [synthetic.make_packed(Q8_0, vocab, HIDDEN, seed=9500 + i, device=dev) for i in range(2)]
        xh = synthetic.make_activations(1, HIDDEN, seed=14, device=dev)
        logits = torch.empty((1, vocab), dtype=torch.bfloat16, device=dev)
        n_h = 64
        _, ev_h = run_region(lambda i: ops.linear_into(xh, heads[i % 2], Q8_0, None, logits, num), n_h, 32)
        hb = linear_bytes(1, vocab, HIDDEN)
        t_heads = [ops.q8_0_tile(w) for w in heads]
        _, ev_ht = run_region(lambda i: ops.linear_tiled_into(xh, t_heads[i % 2], None, None, logits, num), n_h, 32)
        del t_heads
        gh = (torch.rand(HIDDEN, generator=torch.Generator().manual_seed(15)) + 0.5).to(torch.bfloat16).to(dev)
        # the model's final RMSNorm (modeling_qwen3.py:1183; lm_head at :1264 reads its output) folded into the same launch
        _, ev_hn = run_region(lambda i: ops.rmsnorm_linear_into(xh, gh, 1e-6, heads[i % 2], Q8_0, None, logits, num), n_h, 32)
        # greedy token: the arg-max folded into the projection (sngguf_lm_head_argmax) against logits + torch.argmax
        lib = ops.load_library()
        import ctypes
        am_ws = torch.empty(int(lib.sngguf_lm_head_argmax_workspace_bytes(1, vocab)), dtype=torch.uint8, device=dev)
        am_out = torch.empty(1, dtype=torch.int64, device=dev)
        strm = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)

        def head_argmax(i):
            rc = lib.sngguf_lm_head_argmax(ctypes.c_void_p(xh.data_ptr()), 1, ctypes.c_void_p(heads[i % 2].data_ptr()), Q8_0, vocab, HIDDEN,
                                           None, ctypes.c_void_p(am_ws.data_ptr()), ctypes.c_void_p(am_out.data_ptr()), num,
                                           ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
            assert rc == 0, rc

        def head_then_argmax(i):
            ops.linear_into(xh, heads[i % 2], Q8_0, None, logits, num)
            torch.argmax(logits, dim=-1, out=am_out)

        _, ev_am = run_region(head_argmax, n_h, 32)
        _, ev_la = run_region(head_then_argmax, n_h, 32)
        del strm
        result["lm_head"] = {"workload": "Q8_0 lm_head 4096 -> 151936 at M=1, two weight copies alternating",
                             "argmax_fused_us": round(ev_am / n_h * 1e3, 2), "logits_then_torch_argmax_us": round(ev_la / n_h * 1e3, 2),
                             "bytes_per_launch": hb, "avg_launch_us": round(ev_h / n_h * 1e3, 2),
                             "with_final_norm_fused_us": round(ev_hn / n_h * 1e3, 2),
                             "tiled_layout_us": round(ev_ht / n_h * 1e3, 2),
                             "tiled_layout_pct_of_hbm_peak": round(100 * hb / (ev_ht / n_h * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2),
                             "value": round(hb / (ev_h / n_h * 1e-3) / 1e9, 1), "unit": "GB/s",
                             "pct_of_hbm_peak": round(100 * hb / (ev_h / n_h * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2)}
        del heads, logits

    # ---- M = 4096 generation-tower projections on the MFMA GEMM ----------------------------------
    if not args.no_gemm:
        m = 4096
        shapes = [("q", HIDDEN, HIDDEN), ("k", KV, HIDDEN), ("v", KV, HIDDEN), ("o", HIDDEN, HIDDEN),
                  ("gate", INTER, HIDDEN), ("up", INTER, HIDDEN), ("down", HIDDEN, INTER)]
        tower = [[synthetic.make_packed(Q8_0, n, k, seed=5000 + 10 * r + j, device=dev) for j, (_, n, k) in enumerate(shapes)]
                 for r in range(2)]
        xs = {k: synthetic.make_activations(m, k, seed=k, device=dev) for k in (HIDDEN, INTER)}
        ys = {n: torch.empty((m, n), dtype=torch.bfloat16, device=dev) for n in (HIDDEN, KV, INTER)}

        def tower_step(i):
            ws = tower[i % 2]
            for j, (_, n, k) in enumerate(shapes):
                ops.linear_into(xs[k], ws[j], Q8_0, None, ys[n], num)

        def gate_only(i):
            ops.linear_into(xs[HIDDEN], tower[i % 2][4], Q8_0, None, ys[INTER], num)

        gs = args.gemm_steps
        wall, ev = run_region(tower_step, gs, args.gemm_warmup)
        flops = sum(2.0 * m * n * k for _, n, k in shapes)
        tflops = flops / (wall / gs * 1e-3) / 1e12
        _, ev_gate = run_region(gate_only, gs * 2, args.gemm_warmup)
        gate_ms = ev_gate / (gs * 2)

        # GGUFLinear.gemm_policy "two_pass" (opt-in): one dequantize launch to a transient bf16 weight, then the
        # device library's dense GEMM (hipBLASLt through torch.matmul); the default route is tower_ws below
        wtmp = torch.empty(INTER * HIDDEN, dtype=torch.bfloat16, device=dev)

        def two_pass(x, packed, n, k, y):
            w = wtmp[:n * k].view(n, k)
            ops.dequantize_into(packed, Q8_0, w, num)
            torch.matmul(x, w.t(), out=y)

        def tower_two_pass(i):
            ws = tower[i % 2]
            for j, (_, n, k) in enumerate(shapes):
                two_pass(xs[k], ws[j], n, k, ys[n])

        def tower_ws(i):
            wsets = tower[i % 2]
            for j, (_, n, k) in enumerate(shapes):
                ops.linear_ws_into(xs[k], wsets[j], Q8_0, None, ys[n], wtmp, num)

        wall_ws, _ = run_region(tower_ws, gs, args.gemm_warmup)
        _, ev_gate_ws = run_region(lambda i: ops.linear_ws_into(xs[HIDDEN], tower[i % 2][4], Q8_0, None, ys[INTER], wtmp, num),
                                   gs * 2, args.gemm_warmup)
        # the dense tile kernel alone on the gate shape: the weight pass's bf16 output kept, launched as a type-30 weight
        gate_dense = [torch.empty((INTER, HIDDEN), dtype=torch.bfloat16, device=dev) for _ in range(2)]
        for r in range(2):
            ops.dequantize_into(tower[r][4], Q8_0, gate_dense[r], num)
        _, ev_gate_dense = run_region(lambda i: ops.linear_into(xs[HIDDEN], gate_dense[i % 2].view(torch.uint8), 30, None,
                                                                ys[INTER], num), gs * 2, args.gemm_warmup)
        del gate_dense
        dense_ms = ev_gate_dense / (gs * 2)
        wall2, _ = run_region(tower_two_pass, gs, args.gemm_warmup)
        _, ev_gate2 = run_region(lambda i: two_pass(xs[HIDDEN], tower[i % 2][4], INTER, HIDDEN, ys[INTER]), gs * 2, args.gemm_warmup)
        # gemm_policy "resident": the bf16 weights are produced once and kept (2 N K bytes per linear)
        dense = [[torch.empty((n, k), dtype=torch.bfloat16, device=dev) for _, n, k in shapes] for _ in range(2)]
        for r in range(2):
            for j in range(len(shapes)):
                ops.dequantize_into(tower[r][j], Q8_0, dense[r][j], num)

        def tower_resident(i):
            ws = dense[i % 2]
            for j, (_, n, k) in enumerate(shapes):
                ops.linear_ws_into(xs[k], ws[j].view(torch.uint8), ops.BF16, None, ys[n], wtmp, num)

        def tower_resident_device_library(i):
            ws = dense[i % 2]
            for j, (_, n, k) in enumerate(shapes):
                torch.matmul(xs[k], ws[j].t(), out=ys[n])

        wall3, _ = run_region(tower_resident, gs, args.gemm_warmup)
        wall3_dl, _ = run_region(tower_resident_device_library, gs, args.gemm_warmup)
        del dense
        # q | k | v as one [6144, 4096] matrix (rows of the three packed weights one after another, what
        # FusedProjections builds at load): 384 large tiles in one launch instead of 256 + 64 + 64
        qkv = [torch.cat([tower[r][0], tower[r][1], tower[r][2]], dim=0).contiguous() for r in range(2)]
        y_qkv = torch.empty((m, HIDDEN + 2 * KV), dtype=torch.bfloat16, device=dev)
        rest = [(j, n, k) for j, (nm, n, k) in enumerate(shapes) if nm not in ("q", "k", "v")]

        def tower_stacked(i):
            ops.linear_into(xs[HIDDEN], qkv[i % 2], Q8_0, None, y_qkv, num)
            for j, n, k in rest:
                ops.linear_into(xs[k], tower[i % 2][j], Q8_0, None, ys[n], num)

        def tower_stacked_ws(i):
            ops.linear_ws_into(xs[HIDDEN], qkv[i % 2], Q8_0, None, y_qkv, wtmp, num)
            for j, n, k in rest:
                ops.linear_ws_into(xs[k], tower[i % 2][j], Q8_0, None, ys[n], wtmp, num)

        # a few hundred rows (a text prompt): few output tiles, so the workspace route splits K over workgroups
        mid = {}
        for mm in (128, 512):
            xm = {k: synthetic.make_activations(mm, k, seed=40 + k, device=dev) for k in (HIDDEN, INTER)}
            ym = {n: torch.empty((mm, n), dtype=torch.bfloat16, device=dev) for n in (HIDDEN, KV, INTER)}
            row = {}
            for j, (nm, n, k) in enumerate(shapes):
                if nm in ("v", "o", "up"):
                    continue
                _, e_f = run_region(lambda i: ops.linear_into(xm[k], tower[i % 2][j], Q8_0, None, ym[n], num), 16, 4)
                _, e_w = run_region(lambda i: ops.linear_ws_into(xm[k], tower[i % 2][j], Q8_0, None, ym[n], wtmp, num), 16, 4)
                _, e_t = run_region(lambda i: two_pass(xm[k], tower[i % 2][j], n, k, ym[n]), 16, 4)
                row[nm] = {"linear_us": round(e_f / 16 * 1e3, 1), "workspace_us": round(e_w / 16 * 1e3, 1),
                           "two_pass_us": round(e_t / 16 * 1e3, 1)}
            mid[f"M{mm}"] = row
        wall_st, _ = run_region(tower_stacked, gs, args.gemm_warmup)
        wall_st_ws, _ = run_region(tower_stacked_ws, gs, args.gemm_warmup)
        del qkv, y_qkv
        # gate / up / SiLU as Qwen3MLP.forward asks for them at M = 4096: one gated launch of the dense kernel behind the
        # two weight passes (what modality.gated_mlp runs from 2048 rows on) against two workspace launches and the
        # elementwise product on bf16 tensors
        gated = {}
        for mg in (4096, 2048):
            xg = xs[HIDDEN][:mg]
            hg = torch.empty((mg, INTER), dtype=torch.bfloat16, device=dev)
            y_up = torch.empty((mg, INTER), dtype=torch.bfloat16, device=dev)
            ws_g = torch.empty(ops.gate_up_silu_workspace_bytes(INTER, HIDDEN), dtype=torch.uint8, device=dev)

            def gated_fused(i):
                ops.gate_up_silu_ws_into(xg, tower[i % 2][4], tower[i % 2][5], Q8_0, hg, ws_g, num)

            def gated_separate(i):
                ops.linear_ws_into(xg, tower[i % 2][4], Q8_0, None, ys[INTER][:mg], wtmp, num)
                ops.linear_ws_into(xg, tower[i % 2][5], Q8_0, None, y_up, wtmp, num)
                torch.mul(torch.nn.functional.silu(ys[INTER][:mg]), y_up, out=hg)

            _, e_f = run_region(gated_fused, gs * 2, args.gemm_warmup)
            _, e_s = run_region(gated_separate, gs * 2, args.gemm_warmup)
            gated[f"M{mg}"] = {"one_gated_launch_us": round(e_f / (gs * 2) * 1e3, 1),
                               "two_launches_and_product_us": round(e_s / (gs * 2) * 1e3, 1),
                               "tflops": round(4.0 * mg * INTER * HIDDEN / (e_f / (gs * 2) * 1e-3) / 1e12, 1)}
            del hg, y_up, ws_g
        gate_flop = 2.0 * m * INTER * HIDDEN
        gate_tflops = gate_flop / (gate_ms * 1e-3) / 1e12
        dense_tflops = gate_flop / (dense_ms * 1e-3) / 1e12
        tflops_ws = flops / (wall_ws / gs * 1e-3) / 1e12
        tflops_st = flops / (wall_st_ws / gs * 1e-3) / 1e12
        result["gemm"] = {
            "workload": "configs[2]: Q8_0 generation-tower projections over M=4096 image tokens "
                        "(q,o 4096^2; k,v 4096->1024; gate/up 4096->12288; down 12288->4096)",
            "route": "as a model loaded by load_gguf_model runs them: sngguf_linear_ws (weight pass into a pooled bf16 "
                     "workspace + the library's dense tile kernel), q / k / v answered from ONE launch over their stacked "
                     "rows (modality.SharedInputStack: 384 large tiles instead of 256 + 64 + 64), o, gate, up, down one launch each",
            "value": round(tflops_st, 2),
            "unit": "TFLOP/s",
            "steps": gs,
            "warmup": args.gemm_warmup,
            "ms_per_step": round(wall_st_ws / gs, 4),
            "flop_per_step": flops,
            "pct_of_bf16_mfma_peak": round(100 * tflops_st / MFMA_BF16_PEAK_TFLOPS, 2),
            "seven_separate_linears": {
                "what": "the same projections as seven sngguf_linear_ws calls (modules swapped without the loader's q|k|v stack): "
                        "k / v (64 tiles each) with K split four ways over workgroups",
                "value": round(tflops_ws, 2), "unit": "TFLOP/s", "ms_per_step": round(wall_ws / gs, 4),
                "pct_of_bf16_mfma_peak": round(100 * tflops_ws / MFMA_BF16_PEAK_TFLOPS, 2),
            },
            "gate_us": round(ev_gate_ws / (gs * 2) * 1e3, 2),
            "gate_tflops": round(gate_flop / (ev_gate_ws / (gs * 2) * 1e-3) / 1e12, 2),
            "roofline": {
                "kernel": "sngguf::gemm_dense4_kernel (dense bf16, four wavefronts; gate 4096->12288, M=4096; the second "
                          "launch of the route, timed alone on a kept bf16 weight)",
                "bound": "mfma",
                "achieved": round(dense_tflops, 2),
                "peak": MFMA_BF16_PEAK_TFLOPS,
                "unit": "TFLOP/s",
                "frac": round(dense_tflops / MFMA_BF16_PEAK_TFLOPS, 4),
                "traffic": MEASURED_TRAFFIC["gemm_dense_gate_m4096"],
                "flop_per_launch": gate_flop,
                "avg_launch_us": round(dense_ms * 1e3, 2),
            },
            "fused": {
                "what": "sngguf_linear: the Q8_0 decode inside the tile kernel (no workspace), the route of callers that "
                        "pass none",
                "value": round(tflops, 2), "unit": "TFLOP/s", "ms_per_step": round(wall / gs, 4),
                "pct_of_bf16_mfma_peak": round(100 * tflops / MFMA_BF16_PEAK_TFLOPS, 2),
                "roofline": {
                    "kernel": "sngguf::gemm_tile_kernel<Q8_0, upstream_fp16> (gate 4096->12288, M=4096)",
                    "bound": "mfma", "achieved": round(gate_tflops, 2), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(gate_tflops / MFMA_BF16_PEAK_TFLOPS, 4),
                    "traffic": MEASURED_TRAFFIC["gemm_gate_m4096"],
                    "flop_per_launch": gate_flop, "avg_launch_us": round(gate_ms * 1e3, 2),
                },
            },
            "two_pass": {
                "what": "same tower as sngguf dequantize (packed -> bf16, transient) + dense bf16 GEMM of the device "
                        "library (GGUFLinear.gemm_policy 'two_pass', opt-in)",
                "value": round(flops / (wall2 / gs * 1e-3) / 1e12, 2), "unit": "TFLOP/s",
                "ms_per_step": round(wall2 / gs, 4),
                "pct_of_bf16_mfma_peak": round(100 * flops / (wall2 / gs * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 2),
                "gate_us": round(ev_gate2 / (gs * 2) * 1e3, 2),
                "gate_tflops": round(2.0 * m * INTER * HIDDEN / (ev_gate2 / (gs * 2) * 1e-3) / 1e12, 2),
            },
            "stacked_qkv": {
                "what": "the same tower with q, k and v as one stacked [6144, 4096] weight (one launch of 384 large tiles "
                        "instead of 256 + 64 + 64; k / v alone have too few tiles for the large-tile kernel), fused route "
                        "and workspace route",
                "value": round(flops / (wall_st / gs * 1e-3) / 1e12, 2), "unit": "TFLOP/s", "ms_per_step": round(wall_st / gs, 4),
                "pct_of_bf16_mfma_peak": round(100 * flops / (wall_st / gs * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 2),
                "workspace_value": round(flops / (wall_st_ws / gs * 1e-3) / 1e12, 2),
                "workspace_ms_per_step": round(wall_st_ws / gs, 4),
                "workspace_pct_of_bf16_mfma_peak": round(100 * flops / (wall_st_ws / gs * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 2),
            },
            "gated_pair": {
                "what": "silu(gate_proj(x)) * up_proj(x), 4096 -> 12288: sngguf_gate_up_silu_ws (two weight passes into one "
                        "interleaved workspace + ONE dense launch with the gated epilogue; the projection outputs are never "
                        "written) against sngguf_linear_ws twice + the product on bf16 tensors",
                **gated,
            },
            "mid_rows": {
                "what": "one projection at 128 and 512 rows (q 4096^2, k 4096->1024, gate 4096->12288, down 12288->4096): "
                        "sngguf_linear (large-tile kernel, few tiles), sngguf_linear_ws (K split over workgroups, fp32 partial "
                        "sums in the workspace) and dequantize + device-library GEMM",
                **mid,
            },
            "resident": {
                "what": "gemm_policy 'resident': the bf16 weights written once by sngguf dequantize and kept "
                        "(2 N K bytes per linear), every call is the library's dense tile kernel alone (sngguf_linear_ws on "
                        "BF16 rows: K split over workgroups for k / v); device_library_*: torch.matmul on the same kept weights",
                "value": round(flops / (wall3 / gs * 1e-3) / 1e12, 2), "unit": "TFLOP/s", "ms_per_step": round(wall3 / gs, 4),
                "pct_of_bf16_mfma_peak": round(100 * flops / (wall3 / gs * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 2),
                "device_library_value": round(flops / (wall3_dl / gs * 1e-3) / 1e12, 2),
                "device_library_ms_per_step": round(wall3_dl / gs, 4),
            },
        }
        del tower, xs, ys, wtmp

    # ---- standalone dequantize (the reference's dequantize_gguf_tensor): packed [12288, 4096] -> fp16 -----------
    if not args.no_extra:
        deq = {}
        for qt, name in ((Q8_0, "Q8_0"), (Q4_K, "Q4_K"), (Q6_K, "Q6_K")):
            srcs = [synthetic.make_packed(qt, INTER, HIDDEN, seed=3000 + i, device=dev) for i in range(8)]
            out = torch.empty((INTER, HIDDEN), dtype=torch.float16, device=dev)

            def deq_step(i):
                ops.dequantize_into(srcs[i % 8], qt, out, num)

            n_deq = 64
            wall, ev = run_region(deq_step, n_deq, 8)
            nbytes = packed_bytes(qt, INTER, HIDDEN) + 2 * INTER * HIDDEN
            gbps = nbytes / (ev / n_deq * 1e-3) / 1e9
            deq[name] = {"value": round(gbps, 1), "unit": "GB/s", "us": round(ev / n_deq * 1e3, 2),
                         "pct_of_hbm_peak": round(100 * gbps / HBM_PEAK_GBPS, 2), "bytes": nbytes}
            del srcs, out
        deq["workload"] = ("packed [12288, 4096] -> fp16, bytes = packed read + fp16 written; the 100 MB output is "
                           "rewritten every launch and fits the 256 MB last-level cache")
        result["dequantize"] = deq

    # ---- configs[3]: K-quant mix (Q4_K q/k/v/o/gate/up, Q6_K down) at M = 1, 16 and 4096 -----------------
    if not args.no_extra:
        klayers = []
        for i in range(L):
            klayers.append((synthetic.make_packed(Q4_K, INTER, HIDDEN, seed=2000 + 3 * i, device=dev),
                            synthetic.make_packed(Q4_K, INTER, HIDDEN, seed=2001 + 3 * i, device=dev),
                            synthetic.make_packed(Q6_K, HIDDEN, INTER, seed=2002 + 3 * i, device=dev)))
        kq = {}
        for m in (1, 16):
            k2 = max(64, K // 4)
            wall, ev, gu, dn = mlp_leg(m, k2, min(W, 16), klayers, Q4_K, Q6_K)
            nbytes = mlp_bytes(m, Q4_K, Q6_K)
            gbps = nbytes / (wall / k2 * 1e-3) / 1e9
            kq[f"mlp_M{m}"] = {"value": round(gbps, 1), "unit": "GB/s", "pct_of_hbm_peak": round(100 * gbps / HBM_PEAK_GBPS, 2),
                               "bytes_per_step": nbytes, "ms_per_step": round(wall / k2, 6),
                               "gate_up_us": round(gu * 1e3, 3), "down_us": round(dn * 1e3, 3)}
            if m == 1 and ops.mlp_decode_fits(Q4_K, Q6_K, 1, HIDDEN, INTER):
                # the route modality.gated_mlp takes for one or two rows; the two launches stay beside it
                wall1k, _ = mlp_one_launch_leg(1, k2, min(W, 16), klayers, Q4_K, Q6_K)
                g1 = nbytes / (wall1k / k2 * 1e-3) / 1e9
                kq["mlp_M1"] = {"what": "sngguf_mlp_decode, one launch", "value": round(g1, 1), "unit": "GB/s",
                                "pct_of_hbm_peak": round(100 * g1 / HBM_PEAK_GBPS, 2), "bytes_per_step": nbytes,
                                "ms_per_step": round(wall1k / k2, 6), "two_launches": kq["mlp_M1"]}
        # post_attention_layernorm in front of the Q4_K gate/up pair at M = 1: one torch rms_norm launch + the pair,
        # against the norm folded into the pair's launch
        xk = synthetic.make_activations(1, HIDDEN, seed=21, device=dev)
        hk = torch.empty((1, INTER), dtype=torch.bfloat16, device=dev)
        gk = (torch.rand(HIDDEN, generator=torch.Generator().manual_seed(22)) + 0.5).to(torch.bfloat16).to(dev)

        def kq_norm_separate(i):
            nk = torch.nn.functional.rms_norm(xk, (HIDDEN,), gk, 1e-6)
            ops.gate_up_silu_into(nk, klayers[i % L][0], klayers[i % L][1], Q4_K, hk, num)

        def kq_norm_fused(i):
            ops.rmsnorm_gate_up_silu_into(xk, gk, 1e-6, klayers[i % L][0], klayers[i % L][1], Q4_K, hk, num)

        kn = max(64, K // 4)
        wall_ns, _ = run_region(kq_norm_separate, kn, min(W, 16))
        wall_nf, _ = run_region(kq_norm_fused, kn, min(W, 16))
        kq["gate_up_M1_with_norm"] = {"separate_rms_norm_us": round(wall_ns / kn * 1e3, 2), "fused_us": round(wall_nf / kn * 1e3, 2)}
        del klayers
        if not args.no_gemm:
            m = 4096
            kshapes = [("q", HIDDEN, HIDDEN, Q4_K), ("k", KV, HIDDEN, Q4_K), ("v", KV, HIDDEN, Q4_K), ("o", HIDDEN, HIDDEN, Q4_K),
                       ("gate", INTER, HIDDEN, Q4_K), ("up", INTER, HIDDEN, Q4_K), ("down", HIDDEN, INTER, Q6_K)]
            ktower = [[synthetic.make_packed(qt, n, k, seed=6000 + 10 * r + j, device=dev) for j, (_, n, k, qt) in enumerate(kshapes)]
                      for r in range(2)]
            xs = {k: synthetic.make_activations(m, k, seed=k, device=dev) for k in (HIDDEN, INTER)}
            ys = {n: torch.empty((m, n), dtype=torch.bfloat16, device=dev) for n in (HIDDEN, KV, INTER)}

            def ktower_step(i):
                ws = ktower[i % 2]
                for j, (_, n, k, qt) in enumerate(kshapes):
                    ops.linear_into(xs[k], ws[j], qt, None, ys[n], num)

            gs = max(4, args.gemm_steps // 2)
            wall, ev = run_region(ktower_step, gs, max(2, args.gemm_warmup // 2))
            flops = sum(2.0 * m * n * k for _, n, k, _ in kshapes)
            tflops = flops / (wall / gs * 1e-3) / 1e12
            kq["tower_M4096_fused"] = {"what": "sngguf_linear: Q4_K on the fused large-tile kernel, Q6_K on the 128-tile kernel",
                                       "value": round(tflops, 2), "unit": "TFLOP/s", "ms_per_step": round(wall / gs, 4),
                                       "pct_of_bf16_mfma_peak": round(100 * tflops / MFMA_BF16_PEAK_TFLOPS, 2)}
            kws = torch.empty(INTER * HIDDEN, dtype=torch.bfloat16, device=dev)

            def ktower_ws(i):
                wsets = ktower[i % 2]
                for j, (_, n, k, qt) in enumerate(kshapes):
                    ops.linear_ws_into(xs[k], wsets[j], qt, None, ys[n], kws, num)

            wall_kws, _ = run_region(ktower_ws, gs, max(2, args.gemm_warmup // 2))
            tf_kws = flops / (wall_kws / gs * 1e-3) / 1e12
            kq["tower_M4096"] = {"what": "sngguf_linear_ws (weight pass + dense tile kernel), the module's route beyond 64 rows",
                                 "value": round(tf_kws, 2), "unit": "TFLOP/s", "ms_per_step": round(wall_kws / gs, 4),
                                 "pct_of_bf16_mfma_peak": round(100 * tf_kws / MFMA_BF16_PEAK_TFLOPS, 2)}
            del kws
            del ktower, xs, ys
        kq["workload"] = ("configs[3]: Q4_K for q/k/v/o/gate/up, Q6_K for down; decode MLP at M=1,16 "
                          "(GB/s over packed weights + activations) and the 7 tower projections at M=4096")
        result["k_quants"] = kq

    # ---- configs[4]: one MoT layer, 512 text rows -> understanding weights, 4096 image rows -> generation
    # weights, each of the 7 linears through the modality-grouped launcher (Q8_0) ---------------------------
    if not args.no_extra and not args.no_gemm:
        n_text, m = 512, 512 + 4096
        shapes = [("q", HIDDEN, HIDDEN), ("k", KV, HIDDEN), ("v", KV, HIDDEN), ("o", HIDDEN, HIDDEN),
                  ("gate", INTER, HIDDEN), ("up", INTER, HIDDEN), ("down", HIDDEN, INTER)]
        und = [synthetic.make_packed(Q8_0, n, k, seed=7000 + j, device=dev) for j, (_, n, k) in enumerate(shapes)]
        gen = [synthetic.make_packed(Q8_0, n, k, seed=7100 + j, device=dev) for j, (_, n, k) in enumerate(shapes)]
        xs = {k: synthetic.make_activations(m, k, seed=k + 1, device=dev) for k in (HIDDEN, INTER)}
        ys = {n: torch.empty((m, n), dtype=torch.bfloat16, device=dev) for n in (HIDDEN, KV, INTER)}

        def layer_step(i):
            for j, (_, n, k) in enumerate(shapes):
                ops.grouped_linear_into(xs[k], None, n_text, und[j], Q8_0, gen[j], Q8_0, None, None, ys[n], None, num)

        gs = max(4, args.gemm_steps // 2)
        wall, ev = run_region(layer_step, gs, max(2, args.gemm_warmup // 2))
        flops = sum(2.0 * m * n * k for _, n, k in shapes)
        tflops = flops / (wall / gs * 1e-3) / 1e12
        wtmp = torch.empty(INTER * HIDDEN, dtype=torch.bfloat16, device=dev)

        def layer_two_pass(i):
            for j, (_, n, k) in enumerate(shapes):
                for packed, lo, hi in ((und[j], 0, n_text), (gen[j], n_text, m)):
                    w = wtmp[:n * k].view(n, k)
                    ops.dequantize_into(packed, Q8_0, w, num)
                    torch.matmul(xs[k][lo:hi], w.t(), out=ys[n][lo:hi])

        wall2, _ = run_region(layer_two_pass, gs, max(2, args.gemm_warmup // 2))
        dws = torch.empty(2 * INTER * HIDDEN, dtype=torch.bfloat16, device=dev)

        def layer_ws(i):
            for j, (_, n, k) in enumerate(shapes):
                ops.grouped_linear_ws_into(xs[k], None, n_text, und[j], Q8_0, gen[j], Q8_0, None, None, ys[n], None, dws, num)

        wall_gws, _ = run_region(layer_ws, gs, max(2, args.gemm_warmup // 2))
        del dws
        tflops_gws = flops / (wall_gws / gs * 1e-3) / 1e12
        result["grouped_layer"] = {
            "workload": "configs[4], one of the 36 layers: 512 text rows -> understanding weights, 4096 image rows -> "
                        "generation weights, 7 Q8_0 linears through the modality-grouped launcher (contiguous split)",
            "route": "sngguf_grouped_linear_ws (what modality.grouped_linear does with n_text): each group as its own "
                     "workspace-route problem on its row range - K split for the 512 text rows, weight pass + dense tile "
                     "kernel for the 4096 image rows",
            "value": round(tflops_gws, 2), "unit": "TFLOP/s", "ms_per_layer": round(wall_gws / gs, 4),
            "flop_per_layer": flops, "pct_of_bf16_mfma_peak": round(100 * tflops_gws / MFMA_BF16_PEAK_TFLOPS, 2),
            "fused": {
                "what": "sngguf_grouped_linear: one launch of the fused tile kernel over both row groups, no workspace",
                "value": round(tflops, 2), "unit": "TFLOP/s", "ms_per_layer": round(wall / gs, 4),
                "pct_of_bf16_mfma_peak": round(100 * tflops / MFMA_BF16_PEAK_TFLOPS, 2),
            },
            "two_pass": {
                "what": "per group: sngguf dequantize to a transient bf16 weight + the device library's dense bf16 GEMM into "
                        "the group's rows (gemm_policy 'two_pass', opt-in)",
                "value": round(flops / (wall2 / gs * 1e-3) / 1e12, 2), "unit": "TFLOP/s", "ms_per_layer": round(wall2 / gs, 4),
                "pct_of_bf16_mfma_peak": round(100 * flops / (wall2 / gs * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 2),
            },
        }
        del und, gen, wtmp

        # configs[4] as stated: all 36 layers x 2 towers resident (14.76 GB of Q8_0), the 7 grouped linears of every layer
        # in ONE timed region (252 grouped launches), each linear fed the layer's fresh-standing N(0,1) input of its width
        n_layers = 36
        stack = [[(synthetic.make_packed(Q8_0, n, k, seed=20000 + 20 * li + j, device=dev),
                   synthetic.make_packed(Q8_0, n, k, seed=20010 + 20 * li + j, device=dev)) for j, (_, n, k) in enumerate(shapes)]
                 for li in range(n_layers)]
        torch.cuda.synchronize()
        stack_bytes = sum(a.numel() + b.numel() for layer in stack for a, b in layer)
        dws = torch.empty(2 * INTER * HIDDEN, dtype=torch.bfloat16, device=dev)

        def stack_pass(i, ws_route):
            for layer in stack:
                for j, (_, n, k) in enumerate(shapes):
                    wu, wg = layer[j]
                    if ws_route:
                        ops.grouped_linear_ws_into(xs[k], None, n_text, wu, Q8_0, wg, Q8_0, None, None, ys[n], None, dws, num)
                    else:
                        ops.grouped_linear_into(xs[k], None, n_text, wu, Q8_0, wg, Q8_0, None, None, ys[n], None, num)

        stack_flops = n_layers * flops
        wall_sf, _ = run_region(lambda i: stack_pass(i, False), 2, 1)
        wall_sw, _ = run_region(lambda i: stack_pass(i, True), 2, 1)
        result["grouped_stack"] = {
            "workload": "configs[4]: 36 layers x 2 towers in Q8_0 resident in HBM, 512 text rows -> understanding weights + 4096 "
                        "image rows -> generation weights through the modality-grouped launcher, 7 linears per layer, all "
                        "layers in one timed region (linear projections only)",
            "packed_bytes": stack_bytes, "flop_per_pass": stack_flops,
            "route": "sngguf_grouped_linear_ws on one shared workspace (the host layer's default)",
            "value": round(stack_flops / (wall_sw / 2 * 1e-3) / 1e12, 2), "unit": "TFLOP/s", "ms_per_pass": round(wall_sw / 2, 3),
            "pct_of_bf16_mfma_peak": round(100 * stack_flops / (wall_sw / 2 * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 2),
            "fused": {"value": round(stack_flops / (wall_sf / 2 * 1e-3) / 1e12, 2), "unit": "TFLOP/s", "ms_per_pass": round(wall_sf / 2, 3),
                      "pct_of_bf16_mfma_peak": round(100 * stack_flops / (wall_sf / 2 * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 2)},
        }
        del stack, dws, xs, ys

    # ---- layer-offload streaming: decoder layers (understanding tower, 7 Q8_0 linears, 205 MB) kept in pinned
    # host arenas and copied in ahead of their forward on a second stream; the host link bounds this leg ----------
    if not args.no_extra:
        from torch import nn

        from sensenova_u1_amd import GGUFLinear, GGUFParameter, gated_mlp
        from sensenova_u1_amd.layer_offload import ALL_TENSOR_GROUPS, LayerOffloadWrapper

        def qlin(n, k, seed):
            lin = GGUFLinear(k, n, bias=False, compute_dtype=torch.bfloat16)
            lin.weight = GGUFParameter(synthetic.make_packed(Q8_0, n, k, seed=seed, device=dev).cpu(), quant_type=Q8_0)
            return lin

        class StreamLayer(nn.Module):
            def __init__(self, s):
                super().__init__()
                self.q_proj, self.o_proj = qlin(HIDDEN, HIDDEN, s), qlin(HIDDEN, HIDDEN, s + 1)
                self.k_proj, self.v_proj = qlin(KV, HIDDEN, s + 2), qlin(KV, HIDDEN, s + 3)
                self.gate_proj, self.up_proj = qlin(INTER, HIDDEN, s + 4), qlin(INTER, HIDDEN, s + 5)
                self.down_proj = qlin(HIDDEN, INTER, s + 6)

            def forward(self, h):
                q = self.q_proj(h)
                self.k_proj(h)
                self.v_proj(h)
                h = h + self.o_proj(q)
                return h + gated_mlp(h, self.gate_proj, self.up_proj, self.down_proj)

        class StreamModel(nn.Module):
            def __init__(self, n):
                super().__init__()
                self.layers = nn.ModuleList([StreamLayer(8000 + 10 * i) for i in range(n)])

            def forward(self, h):
                for layer in self.layers:
                    h = layer(h)
                return h

        n_sl, passes = 6, 3
        model = StreamModel(n_sl).eval()
        layer_bytes = sum(p.numel() for p in model.layers[0].parameters())
        hs = {m: synthetic.make_activations(m, HIDDEN, seed=13, device=dev) for m in (1, 4096)}

        def timed_passes(fn, h):
            fn(h)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(passes):
                fn(h)
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) / (passes * n_sl) * 1e3

        model.to(dev)
        stream = {f"M{m}": {"resident_ms_per_layer": round(timed_passes(model, h), 3)} for m, h in hs.items()}
        model.to("cpu")
        for prefetch in (0, 2):
            wrapped = LayerOffloadWrapper(model, "layers", dev, prefetch_count=prefetch)
            for m, h in hs.items():
                ms = timed_passes(wrapped, h)
                stream[f"M{m}"][f"prefetch_{prefetch}"] = {"ms_per_layer": round(ms, 3),
                                                           "host_link_GBps": round(layer_bytes / ms / 1e6, 2)}
            if prefetch == 0:
                store = wrapped.store
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                torch.cuda.synchronize()
                e0.record()
                for _ in range(passes):
                    for i in range(n_sl):
                        store.move_to_gpu(i, groups=ALL_TENSOR_GROUPS, non_blocking=True)
                        store.evict_to_cpu(i)
                e1.record()
                torch.cuda.synchronize()
                copy_ms = e0.elapsed_time(e1) / (passes * n_sl)
                slots = sum(store.slots_allocated().values())
            wrapped.teardown()
        result["offload_stream"] = {
            "workload": f"{n_sl} decoder layers (7 Q8_0 linears each, {layer_bytes} packed bytes per layer) held in pinned host "
                        "arenas, one copy per layer into a ring of device slots, forward of the 7 linears per layer at M=1 and "
                        "M=4096; time per layer over whole passes, wall clock; prefetch_0 copies on the compute stream, "
                        "prefetch_2 two layers ahead on a second stream",
            "bytes_per_layer": layer_bytes,
            "copy_only": {"ms_per_layer": round(copy_ms, 3), "GBps": round(layer_bytes / copy_ms / 1e6, 2), "device_slots": slots},
            **stream,
        }
        del model

    # ---- CPU baseline: the oracle's port of GGUFLinear.forward_native on the host cores -----------
    if not args.no_cpu_baseline:
        from oracle import gguf_oracle as go

        gate, up, down = (t.cpu() for t in layers[0])
        x = synthetic.make_activations(1, HIDDEN, seed=7)
        reps, times = 15, []
        go.mlp_forward(x, gate[:256], up[:256], down[:, :256 // 32 * 34], (Q8_0, Q8_0, Q8_0))  # warm torch's thread pool
        for _ in range(reps):
            t0 = time.perf_counter()
            go.mlp_forward(x, gate, up, down, (Q8_0, Q8_0, Q8_0))
            times.append(time.perf_counter() - t0)
        med = sorted(times)[len(times) // 2]
        result["cpu_baseline"] = {
            "value": round(step_bytes / med / 1e9, 3),
            "unit": "GB/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"median of {reps} full M=1 MLP steps (one layer, {step_bytes} algorithmic bytes each): torch-CPU "
                      "block decode -> bf16 cast -> F.linear, as GGUFLinear.forward_native does",
            "ms_per_step": round(med * 1e3, 2),
            "host_cpus": os.cpu_count(),
        }

    print(json.dumps(result))


if __name__ == "__main__":
    main()
