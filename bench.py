#!/usr/bin/env python3
"""Benchmark of the `hip` decode hot path on one MI355X.

Workload (BASELINE.json configs[1]): the Llama-3-8B decode-layer GEMV set at
batch 1 -- per layer fused QKV 6144x4096, O 4096x4096, gate and up 14336x4096
(Q4_K), down 4096x14336 (Q6_K), plus the output head 128256x4096 (Q6_K).  One
"step" is one token's worth: 32 layers + head (129 launches: QKV, O, fused gate+up, down per layer) over
4 841 250 816 bytes of weights, every layer in its own HBM allocation so the
4.8 GB working set rotates far past the 256 MB last-level cache.  Activations
(Q8_0-quantized x ~ N(0,1)) and weights are resident in HBM before timing.

Prints ONE JSON line (see README / DESIGN.md for the fields).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth

# (name, ggml type name, m, k, copies per step)
LAYER_SET = [
    ("attn_qkv", "Q4_K", 6144, 4096),
    ("attn_output", "Q4_K", 4096, 4096),
    ("ffn_gate", "Q4_K", 14336, 4096),
    ("ffn_up", "Q4_K", 14336, 4096),
    ("ffn_down", "Q6_K", 4096, 14336),
]
HEAD = ("output", "Q6_K", 128256, 4096)
N_LAYERS = 32


def algorithmic_bytes(H, tname, m, k):
    """Weights + Q8_0 activations (k int8 + k/32 f32 scales) + f32 output: the
    reference's own GEMV bandwidth convention (cera/src/backend/cpu.rs:7333-7336)."""
    return m * H.row_bytes(H.TYPE_IDS[tname], k) + k + k // 32 * 4 + m * 4


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--seed", type=int, default=20250)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the hot path has no multi-GPU part); "
              "run with --gpus 1", file=sys.stderr)
        return 2

    from cera_amd import hip_api, host_api as H

    ctx = hip_api.Context(0)
    dev_name, n_cu, hbm = ctx.device_info()
    rng = np.random.default_rng(args.seed)
    n_thr = min(16, os.cpu_count() or 1)

    # ---- synthetic weights: one properly quantized layer + head, cloned on device
    t0 = time.time()
    host = {}
    for name, tname, m, k in LAYER_SET + [HEAD]:
        w = rng.standard_normal((m, k), dtype=np.float32)
        w *= np.float32(0.02)
        host[name] = H.quantize(H.TYPE_IDS[tname], w, n_thr)
        del w
    dts = {}   # name -> list of device tensor handles (one per layer)
    for name, tname, m, k in LAYER_SET:
        first = ctx.tensor_upload(H.TYPE_IDS[tname], m, k, host[name])
        dts[name] = [first] + [ctx.tensor_clone(first) for _ in range(N_LAYERS - 1)]
    name, tname, m, k = HEAD
    dts[name] = [ctx.tensor_upload(H.TYPE_IDS[tname], m, k, host[name])]
    gen_s = time.time() - t0

    # ---- activations, quantized on the device, resident before timing
    acts = {}
    for kk in (4096, 14336):
        x = rng.standard_normal(kk, dtype=np.float32)
        dx = ctx.to_device(x)
        dxs, dxq = ctx.malloc(kk // 32 * 4), ctx.malloc(kk)
        ctx.check(ctx.lib.cera_hip_quantize_q8_0_dev(ctx.h, dx, kk, dxs, dxq))
        acts[kk] = (dxs, dxq, x)
    outs = {name: ctx.malloc(m * 4) for name, _, m, _ in LAYER_SET + [HEAD]}
    ctx.sync()

    def make_ops(entries):
        arr = (hip_api.GemvOp * len(entries))()
        for i, (name, layer, k) in enumerate(entries):
            if isinstance(name, tuple):   # fused FFN pair: silu(gate.x) * (up.x) in one launch
                arr[i] = hip_api.GemvOp(dts[name[0]][layer], dts[name[1]][layer], acts[k][0], acts[k][1], outs[name[0]])
            else:
                arr[i] = hip_api.GemvOp(dts[name][layer], None, acts[k][0], acts[k][1], outs[name])
        return arr

    # group A: the dominant kernel (Q4_K 14336x4096 gate/up), B: other Q4_K, C: Q6_K
    # (gate and up run as the fused pair the decode path uses: one launch, both matrices)
    grp_a = make_ops([(("ffn_gate", "ffn_up"), l, 4096) for l in range(N_LAYERS)])
    grp_b = make_ops([(n, l, 4096) for l in range(N_LAYERS) for n in ("attn_qkv", "attn_output")])
    grp_c = make_ops([("ffn_down", l, 14336) for l in range(N_LAYERS)] + [("output", 0, 4096)])
    groups = [("q4k_gate_up", grp_a), ("q4k_qkv_o", grp_b), ("q6k_down_head", grp_c)]
    shape = {n: (t, m, k) for n, t, m, k in LAYER_SET + [HEAD]}
    bytes_of = {n: algorithmic_bytes(H, *shape[n]) for n in shape}
    grp_bytes = {
        "q4k_gate_up": N_LAYERS * (bytes_of["ffn_gate"] + bytes_of["ffn_up"] - 4096 - 512 - 14336 * 4),
        "q4k_qkv_o": N_LAYERS * (bytes_of["attn_qkv"] + bytes_of["attn_output"]),
        "q6k_down_head": N_LAYERS * bytes_of["ffn_down"] + bytes_of["output"],
    }
    step_bytes = sum(grp_bytes.values())
    weight_bytes = sum(N_LAYERS * len(host[n]) for n, *_ in LAYER_SET) + len(host["output"])

    def run_step(events=None):
        for gi, (_, ops) in enumerate(groups):
            ctx.check(ctx.lib.cera_hip_gemv_seq_dev(ctx.h, ops, len(ops)))
            if events is not None:
                ctx.record(events[gi + 1])

    for _ in range(args.warmup):
        run_step()
    ctx.sync()

    # ---- timed region: exactly --steps steps, bracketed by synchronisation
    evs = [[ctx.event() for _ in range(4)] for _ in range(args.steps)]
    ctx.sync()
    t_start = time.perf_counter()
    for s in range(args.steps):
        ctx.record(evs[s][0])
        run_step(evs[s])
    ctx.sync()
    wall = time.perf_counter() - t_start
    grp_ms = {g: 0.0 for g, _ in groups}
    for s in range(args.steps):
        for gi, (g, _) in enumerate(groups):
            grp_ms[g] += ctx.elapsed_ms(evs[s][gi], evs[s][gi + 1])
    ms_per_step = wall * 1e3 / args.steps
    value = step_bytes / (wall / args.steps) / 1e9

    # dominant kernel: the fused Q4_K gate+up GEMV, 2 x (14336 x 4096) per launch, 32 launches per step
    n_launch = len(grp_a) * args.steps
    avg_launch_ms = grp_ms["q4k_gate_up"] / n_launch
    pair_bytes = bytes_of["ffn_gate"] + bytes_of["ffn_up"] - 4096 - 512 - 14336 * 4   # x and y counted once
    ach = pair_bytes / (avg_launch_ms * 1e-3) / 1e9
    roofline = {"bound": "hbm", "kernel": "gemv_kernel<Q4K,1,2,4,2,false> (Q4_K gate+up, 2 x 14336x4096)",
                "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": None,
                "bytes_per_launch": pair_bytes, "avg_launch_us": round(avg_launch_ms * 1e3, 2)}
    per_group = {g: {"GB/s": round(grp_bytes[g] / (grp_ms[g] / args.steps * 1e-3) / 1e9, 1),
                     "ms_per_step": round(grp_ms[g] / args.steps, 4)} for g, _ in groups}

    # ---- correctness spot check of what was just timed (oracle is only the checker)
    cpu_baseline = None
    if not args.no_cpu_baseline:
        from oracle import binding as orc
        name = "attn_output"
        tname, m, k = shape[name]
        y = ctx.download(outs[name], (m,), np.float32)
        ref = orc.gemv(H.TYPE_IDS[tname], host[name], acts[k][2], m, k)
        rel = float(np.abs(y - ref).max() / np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
        assert rel <= 1e-3, f"GPU result of the timed GEMV deviates from the oracle: {rel}"
        # CPU baseline: the restated cera AVX2 int8 path on a bounded sample --
        # whole layers' GEMV sets (QKV, O, gate, up, down), rotating over distinct
        # weight copies so the host LLC does not hold them.
        pool = orc.Pool(n_thr)
        n_copies = 8
        layer_sets = []
        for c in range(n_copies):
            layer_sets.append({n: (host[n] if c == 0 else host[n].copy()) for n, *_ in LAYER_SET})
        ybuf = {n: np.empty(shape[n][1], np.float32) for n, *_ in LAYER_SET}
        layer_bytes = sum(bytes_of[n] for n, *_ in LAYER_SET)
        done_layers = 0
        t_cpu = time.perf_counter()
        while time.perf_counter() - t_cpu < args.cpu_seconds or done_layers < 2:
            ws = layer_sets[done_layers % n_copies]
            for n, tname, m, k in LAYER_SET:
                pool.gemv(H.TYPE_IDS[tname], ws[n], acts[k][2], m, k, ybuf[n])
            done_layers += 1
        cpu_s = time.perf_counter() - t_cpu
        pool.close()
        cpu_baseline = {"value": round(done_layers * layer_bytes / cpu_s / 1e9, 2), "unit": "GB/s",
                        "cores": n_thr, "kind": "port",
                        "sample": f"{done_layers} decode-layer GEMV sets (QKV, O, gate, up Q4_K; down Q6_K; "
                                  f"{layer_bytes} B each) in {cpu_s:.1f} s, restated cera AVX2 int8 path "
                                  f"incl. per-call Q8_0 quantize, {n_copies} rotating weight copies",
                        "avx2": bool(orc.lib().orc_have_avx2())}

    out = {
        "metric": "Q4_K GEMV HBM GB/s (% of peak); Llama-3-8B-arch Q4_K decode tok/s, 1 GPU",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": "Llama-3-8B decode-layer GEMV set, batch 1: 32 x (QKV 6144x4096, O 4096x4096, "
                               "gate+up 14336x4096 Q4_K; down 4096x14336 Q6_K) + head 128256x4096 Q6_K",
                   "launches_per_step": sum(len(o) for _, o in groups), "weight_bytes_per_step": weight_bytes,
                   "algorithmic_bytes_per_step": step_bytes, "w_sigma": 0.02, "seed": args.seed,
                   "distinct_weight_copies": N_LAYERS},
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
        "gemv_only_tok_s_equiv": round(1e3 / ms_per_step, 1),
        "per_group": per_group,
        "roofline": roofline,
        "cpu_baseline": cpu_baseline,
        "device": dev_name, "n_cu": n_cu, "setup_s": round(gen_s, 1),
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
