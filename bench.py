#!/usr/bin/env python3
"""Benchmark of the `hip` decode hot path on one MI355X.

Workload (BASELINE.json configs[1]): the Llama-3-8B decode-layer GEMV set at
batch 1 -- per layer fused QKV 6144x4096, O 4096x4096, gate and up 14336x4096
(Q4_K), down 4096x14336 (Q6_K), plus the output head 128256x4096 (Q6_K).  One
"step" is one token's worth: 32 layers + head (129 launches: QKV, O, fused gate+up, down per layer) over
4 841 250 816 bytes of weights, every layer in its own HBM allocation so the
4.8 GB working set rotates far past the 256 MB last-level cache.  Activations
(Q8_0-quantized x ~ N(0,1)) and weights are resident in HBM before timing.

Prints ONE JSON line: metric / value / unit, the roofline of the dominant kernel, the CPU baseline,
and (unless disabled) end-to-end, flash-decode and prefill-GEMM measurements.
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
# HBM bytes per launch of the fused Q4_K gate+up GEMV from hardware counters (FETCH_SIZE + WRITE_SIZE,
# each scaled by what the same counter reads for this library's 1 GiB copy kernel; the two passes run
# `bench.py --pmc-probe` under rocprofv3 --pmc, summary in profiles/gemv_q4k_gate_up_hbm_traffic_pmc.txt).
# It is a recorded measurement of this kernel configuration, not taken live: counters need the profiler.
GATE_UP_TRAFFIC_BYTES = 66_328_548
GATE_UP_TRAFFIC_KERNEL = "gemv_kernel<Q4K,1,2,4,2,false>"

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


def host_cpu_info():
    """CPU model and physical / logical core counts of the host the CPU baseline ran on."""
    model, cores = "unknown", set()
    try:
        phys = core = None
        for line in open("/proc/cpuinfo"):
            key, _, val = line.partition(":")
            key, val = key.strip(), val.strip()
            if key == "model name":
                model = val
            elif key == "physical id":
                phys = val
            elif key == "core id":
                core = val
            elif not key and phys is not None:
                cores.add((phys, core))
                phys = core = None
    except OSError:
        pass
    return {"cpu_model": model, "physical_cores": len(cores) or None, "logical_cores": os.cpu_count()}


def measure_attention(ctx, hip_api, rng):
    """BASELINE.json configs[3]: GQA flash-decode, 32 q heads / 8 kv heads / head_dim 128, f32 KV
    resident in HBM in the kernel's head-major layout; bytes = K + V read once."""
    n_heads, n_kv, hd = 32, 8, 128
    out = []
    max_l = 131072
    chunk = rng.standard_normal(1 << 22, dtype=np.float32)            # 16 MiB of N(0,1), tiled over the cache
    kv_bytes = n_kv * max_l * hd * 4
    dk, dv = ctx.malloc(kv_bytes), ctx.malloc(kv_bytes)
    dchunk = ctx.to_device(chunk)
    for off in range(0, kv_bytes, chunk.nbytes):
        ctx.check(ctx.lib.cera_hip_copy_dev(ctx.h, dk + off, dchunk, chunk.nbytes))
        ctx.check(ctx.lib.cera_hip_copy_dev(ctx.h, dv + off, dchunk, chunk.nbytes))
    dq = ctx.to_device(rng.standard_normal(n_heads * hd, dtype=np.float32))
    dout = ctx.malloc(n_heads * hd * 4)
    scale = 1.0 / np.sqrt(hd)
    for L in (512, 4096, 32768, 131072):
        # each context length gets its own cache stride = L, as a model with max_seq_len = L would
        call = lambda: ctx.check(ctx.lib.cera_hip_attn_decode_dev(ctx.h, dq, dk, dv, n_heads, n_kv, hd, L, L,
                                                                  C.c_float(scale), 0, dout))
        iters = 200 if L <= 4096 else 50
        for _ in range(5):
            call()
        e0, e1 = ctx.event(), ctx.event()
        ctx.record(e0)
        for _ in range(iters):
            call()
        ctx.record(e1)
        ctx.sync()
        us = ctx.elapsed_ms(e0, e1) * 1e3 / iters
        nbytes = 2 * n_kv * L * hd * 4 + 2 * n_heads * hd * 4
        # below ~32k the K/V working set fits the 256 MB last-level cache when launched back to back
        out.append({"context": L, "us_per_call": round(us, 2), "GB/s": round(nbytes / us / 1e3, 1),
                    "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                    "cache_resident": 2 * n_kv * L * hd * 4 <= 256 << 20})
    # the same contexts over an f16 KV cache (KvCompression::F16): half the bytes per position
    chunk16 = chunk.astype(np.float16)
    dchunk16 = ctx.to_device(chunk16.view(np.uint16))
    for off in range(0, kv_bytes // 2, chunk16.nbytes):
        ctx.check(ctx.lib.cera_hip_copy_dev(ctx.h, dk + off, dchunk16, chunk16.nbytes))
        ctx.check(ctx.lib.cera_hip_copy_dev(ctx.h, dv + off, dchunk16, chunk16.nbytes))
    for L in (4096, 32768, 131072):
        call = lambda: ctx.check(ctx.lib.cera_hip_attn_decode_f16_dev(ctx.h, dq, dk, dv, n_heads, n_kv, hd, L, L,
                                                                      C.c_float(scale), 0, dout))
        iters = 200 if L <= 4096 else 50
        for _ in range(5):
            call()
        e0, e1 = ctx.event(), ctx.event()
        ctx.record(e0)
        for _ in range(iters):
            call()
        ctx.record(e1)
        ctx.sync()
        us = ctx.elapsed_ms(e0, e1) * 1e3 / iters
        nbytes = 2 * n_kv * L * hd * 2 + 2 * n_heads * hd * 4
        out.append({"context": L, "kv": "f16", "us_per_call": round(us, 2), "GB/s": round(nbytes / us / 1e3, 1),
                    "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                    "cache_resident": 2 * n_kv * L * hd * 2 <= 256 << 20})
    for d in (dk, dv, dchunk, dchunk16, dq, dout):
        ctx.free(d)
    return out


def measure_gemm(ctx, H, dts, shape, rng):
    """BASELINE.json configs[2]: prefill GEMM out[N][M] = W_q . Q8_0(X[M][K]) on the matrix cores, activation
    quantization included in the timed call."""
    INT8_PEAK_TOPS = 5000.0  # MI355X published dense int8 MFMA rate
    F16_PEAK_TOPS = 2500.0   # ... and dense f16
    res = []
    for name in ("ffn_gate", "ffn_down"):
        tname, n_out, k = shape[name]
        for m_tok in (128, 512, 2048):
            dx = ctx.to_device(rng.standard_normal((m_tok, k), dtype=np.float32))
            dout = ctx.malloc(n_out * m_tok * 4)
            call = lambda: ctx.check(ctx.lib.cera_hip_gemm_dev(ctx.h, dts[name][0], dx, m_tok, dout))
            for _ in range(3):
                call()
            e0, e1 = ctx.event(), ctx.event()
            iters = 20
            ctx.record(e0)
            for _ in range(iters):
                call()
            ctx.record(e1)
            ctx.sync()
            us = ctx.elapsed_ms(e0, e1) * 1e3 / iters
            tops = 2.0 * m_tok * n_out * k / us / 1e6
            # Q6_K's block dots run on the f16 matrix cores (2.5 PFLOP/s dense), the rest on int8 (5 POP/s)
            peak_key, peak = ("frac_of_f16_mfma_peak", F16_PEAK_TOPS) if tname == "Q6_K" else ("frac_of_int8_mfma_peak", INT8_PEAK_TOPS)
            res.append({"weight": f"{name} {tname} {n_out}x{k}", "tokens": m_tok, "us_per_call": round(us, 1),
                        "TOP/s": round(tops, 1), peak_key: round(tops / peak, 4)})
            ctx.free(dx)
            ctx.free(dout)
    return res


def measure_e2e(seed: int, n_thr: int):
    """BASELINE.json configs[4]: random-init Llama-3-8B-architecture GGUF written to a temp file, loaded
    through the GGUF reader + HipLlamaModel, 512-token prefill + 256 greedy tokens."""
    import tempfile
    from cera_amd import host_api as H, llama_api, synth
    cfg = dict(synth.LLAMA3_8B, max_seq_len=1024)
    with tempfile.TemporaryDirectory() as td:
        path = os.path.join(td, "llama3_8b_synth.gguf")
        t0 = time.time()
        H.synth_llama_gguf(path, cfg, seed=seed, n_threads=n_thr, explicit_head_dim=False)
        gen_s = time.time() - t0
        size = os.path.getsize(path)
        t0 = time.time()
        m = llama_api.HipLlama(path, context_size=1024)
        load_s = time.time() - t0
    prompt = np.random.default_rng(seed).integers(0, cfg["vocab"], 512).astype(np.uint32)
    m.generate_greedy(prompt, 8)                      # warm-up (first-use allocations)
    runs = []
    for _ in range(3):
        m.truncate_kv(0)
        toks, tp, td_ = m.generate_greedy(prompt, 256, ubatch=512)
        runs.append((512 / tp, 255 / td_))
    # short batches (a few new tokens of a chat turn, the verification pass of speculative decoding):
    # all-position logits of n tokens on top of the 512-token context, weights streamed once per pass
    short = []
    for n_tok in (1, 2, 4, 8):
        toks_n = prompt[:n_tok]
        best = 1e9
        for _ in range(5):
            m.truncate_kv(512)
            t0 = time.perf_counter()
            m.forward_prefill_logits_all(toks_n, 512)
            best = min(best, time.perf_counter() - t0)
        short.append({"tokens": n_tok, "ms_per_pass": round(best * 1e3, 2), "ms_per_token": round(best * 1e3 / n_tok, 2)})
    mem = m.gpu_memory_bytes
    m.close()
    runs.sort(key=lambda r: r[1])
    pf, dec = runs[len(runs) // 2]
    weight_bytes_per_token = 4_875_853_824   # every projection + head read once per token
    return {"workload": "random-init Llama-3-8B arch GGUF (Q4_K_M-style mix), prefill 512 + greedy 256, batch 1, "
                        "host API calls included",
            "decode_tok_s": round(dec, 1), "prefill_tok_s": round(pf, 1),
            "decode_weight_GB/s": round(dec * weight_bytes_per_token / 1e9, 1),
            "decode_frac_of_hbm_peak": round(dec * weight_bytes_per_token / 1e9 / HBM_PEAK_GBS, 4),
            "gguf_bytes": size, "gpu_memory_bytes": mem, "gguf_write_s": round(gen_s, 1), "load_s": round(load_s, 1),
            "runs": 3, "statistic": "median by decode rate",
            "all_logits_short_batch": short}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--seed", type=int, default=20250)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--weight-copies", type=int, default=N_LAYERS,
                    help="distinct HBM copies of the layer weights the step rotates over (default: one per layer; "
                         "fewer lets the last-level cache hold them, which is NOT the reported configuration)")
    ap.add_argument("--no-e2e", action="store_true", help="skip the end-to-end model run (prefill 512 + greedy 256)")
    ap.add_argument("--no-extras", action="store_true", help="skip the flash-decode and prefill-GEMM side measurements")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="run only a 1 GiB copy kernel and one step of the fused gate+up GEMVs, for a "
                         "hardware-counter pass under rocprofv3 --pmc; prints no JSON")
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
        copies = [first] + [ctx.tensor_clone(first) for _ in range(max(1, min(N_LAYERS, args.weight_copies)) - 1)]
        dts[name] = [copies[l % len(copies)] for l in range(N_LAYERS)]
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

    if args.pmc_probe:
        n = 1 << 30
        src, dst = ctx.malloc(n), ctx.malloc(n)
        ctx.check(ctx.lib.cera_hip_copy_kernel(ctx.h, dst, src, n))   # first touch
        for _ in range(3):
            ctx.check(ctx.lib.cera_hip_copy_kernel(ctx.h, dst, src, n))
        for _ in range(2):
            ctx.check(ctx.lib.cera_hip_gemv_seq_dev(ctx.h, grp_a, len(grp_a)))
            ctx.check(ctx.lib.cera_hip_gemv_seq_dev(ctx.h, grp_c, len(grp_c)))
        ctx.sync()
        print(f"pmc probe done: copy kernel {n} B read + {n} B written per launch; fused gate+up "
              f"{grp_bytes['q4k_gate_up'] // N_LAYERS} algorithmic B per launch", file=sys.stderr)
        return 0

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
                "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": GATE_UP_TRAFFIC_BYTES,
                "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE passes over bench.py --pmc-probe, "
                                  "calibrated on a 1 GiB copy kernel (recorded, see profiles/)",
                "bytes_per_launch": pair_bytes, "avg_launch_us": round(avg_launch_ms * 1e3, 2)}
    per_group = {g: {"GB/s": round(grp_bytes[g] / (grp_ms[g] / args.steps * 1e-3) / 1e9, 1),
                     "ms_per_step": round(grp_ms[g] / args.steps, 4)} for g, _ in groups}

    # ---- the Q8_0 activation quantizer on its own (the reference re-quantizes per GEMV call,
    # cpu.rs:787-790): kernel time per call, and the set's rate with one quantize per GEMV folded in
    quant_us = {}
    for kk in (4096, 14336):
        dxf = ctx.to_device(acts[kk][2])
        qcall = lambda: ctx.check(ctx.lib.cera_hip_quantize_q8_0_dev(ctx.h, dxf, kk, acts[kk][0], acts[kk][1]))
        for _ in range(5):
            qcall()
        e0, e1 = ctx.event(), ctx.event()
        ctx.record(e0)
        for _ in range(200):
            qcall()
        ctx.record(e1)
        ctx.sync()
        quant_us[kk] = ctx.elapsed_ms(e0, e1) * 1e3 / 200
        ctx.free(dxf)
    quant_ms_per_step = (N_LAYERS * (4 * quant_us[4096] + quant_us[14336]) + quant_us[4096]) * 1e-3
    quantize = {"k4096_us_per_call": round(quant_us[4096], 2), "k14336_us_per_call": round(quant_us[14336], 2),
                "calls_per_step": N_LAYERS * 5 + 1,
                "set_incl_quantize_GB/s": round(step_bytes / ((ms_per_step + quant_ms_per_step) * 1e-3) / 1e9, 1),
                "note": "back-to-back launches of the standalone kernel; the decode path fuses three of the "
                        "five per-layer quantizations into the producing kernels"}

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
                        "avx2": bool(orc.lib().orc_have_avx2()), **host_cpu_info()}

    extras = {}
    if not args.no_extras:
        extras["flash_decode"] = measure_attention(ctx, hip_api, rng)
        extras["prefill_gemm"] = measure_gemm(ctx, H, dts, shape, rng)
    e2e = None if args.no_e2e else measure_e2e(args.seed, n_thr)

    out = {
        "metric": "Q4_K GEMV HBM GB/s (% of peak); Llama-3-8B-arch Q4_K decode tok/s, 1 GPU",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": "Llama-3-8B decode-layer GEMV set, batch 1: 32 x (QKV 6144x4096, O 4096x4096, "
                               "gate+up 14336x4096 Q4_K; down 4096x14336 Q6_K) + head 128256x4096 Q6_K",
                   "launches_per_step": sum(len(o) for _, o in groups), "weight_bytes_per_step": weight_bytes,
                   "algorithmic_bytes_per_step": step_bytes, "w_sigma": 0.02, "seed": args.seed,
                   "distinct_weight_copies": max(1, min(N_LAYERS, args.weight_copies))},
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
        "gemv_only_tok_s_equiv": round(1e3 / ms_per_step, 1),
        "per_group": per_group,
        "quantize": quantize,
        "roofline": roofline,
        "cpu_baseline": cpu_baseline,
        "e2e": e2e,
        **extras,
        "device": dev_name, "n_cu": n_cu, "setup_s": round(gen_s, 1),
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
