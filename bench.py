#!/usr/bin/env python3
"""Benchmark of the `hip` decode hot path on one MI355X.

Workload (BASELINE.json configs[1]): the Llama-3-8B decode-layer GEMV set at
batch 1 -- per layer fused QKV 6144x4096, O 4096x4096, gate and up 14336x4096
(Q4_K), down 4096x14336 (Q6_K), plus the output head 128256x4096 (Q6_K).  One
"step" is one token's worth, in the order and with the launches the decode path issues: per
layer Q|K|V (rmsnorm + Q8_0 of its input inside the launch), O (+ residual), gate|up (rmsnorm +
Q8_0 in, SwiGLU + Q8_0 out), down (+ residual); then rmsnorm + Q8_0 and the head: 130 launches
over 4 841 250 816 bytes of weights, every layer in its own HBM allocation so the 4.8 GB
working set rotates far past the 256 MB last-level cache.  Weights and the f32 / Q8_0 inputs
(x ~ N(0,1)) are resident in HBM before timing.

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
GATE_UP_TRAFFIC_BYTES = 66_481_099
GATE_UP_KERNEL = "row_gemv_kernel<Q4K,16,4,true,2,true,1,4096>"
# Average duration of that kernel among the other launches of a decode step, from the rocprofv3 kernel trace
# of the whole default run (profiles/gemv_decode_set_llama3_8b_kernel_trace.txt): a recorded figure, kept
# beside the live back-to-back one because events around a single launch inside a step would time the
# launch gap, not the kernel.
GATE_UP_IN_STEP_US = 14.24
# Average duration rocprofv3 reports for the same kernel over `bench.py --roofline-probe` (back-to-back launches only,
# profiles/gemv_gate_up_back_to_back_kernel_trace.txt).  Consecutive launches overlap by a ramp and a tail, so a
# launch's own start-to-end duration is longer than the time per launch the events measure (wall time / launches).
GATE_UP_TRACE_BACK_TO_BACK_US = 14.15

# (name, ggml type name, m, k, copies per step)
LAYER_SET = [
    ("attn_qkv", "Q4_K", 6144, 4096),
    ("attn_output", "Q4_K", 4096, 4096),
    ("ffn_gate", "Q4_K", 14336, 4096),
    ("ffn_up", "Q4_K", 14336, 4096),
    ("ffn_down", "Q6_K", 4096, 14336),
]
HEAD = ("output", "Q6_K", 128256, 4096)
CONFIG1 = ("config1_q4_0", "Q4_0", 4096, 4096)   # BASELINE.json configs[0]: the reference's CPU-runnable GEMV case
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


def _time_calls(ctx, calls, iters, warm=3):
    """Average microseconds per call of `calls[i % len(calls)]()` over `iters` calls (HIP events)."""
    for i in range(warm):
        calls[i % len(calls)]()
    e0, e1 = ctx.event(), ctx.event()
    ctx.record(e0)
    for i in range(iters):
        calls[i % len(calls)]()
    ctx.record(e1)
    ctx.sync()
    return ctx.elapsed_ms(e0, e1) * 1e3 / iters


def measure_attention(ctx, hip_api, rng):
    """BASELINE.json configs[3]: GQA flash-decode, 32 q heads / 8 kv heads / head_dim 128, KV resident in
    HBM in the kernel's head-major layout; bytes = K + V read once.  Every context length rotates over
    distinct caches (about 1 GiB in all) so each call streams from HBM, not from the 256 MB last-level
    cache; the back-to-back rate on ONE cache is kept beside it where that cache fits the LLC."""
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

    def rows(fn, esz, lengths, tag):
        for L in lengths:
            # each context length gets its own cache stride = L, as a model with max_seq_len = L would;
            # cache i of the rotation starts i * (bytes of one cache) into the two big buffers
            one = n_kv * L * hd * esz
            n_rot = max(1, min(kv_bytes // one, -(-(1 << 30) // (2 * one))))
            calls = [(lambda o=i * one: ctx.check(fn(ctx.h, dq, dk + o, dv + o, n_heads, n_kv, hd, L, L, C.c_float(scale), 0, dout)))
                     for i in range(n_rot)]
            iters = 256 if L <= 4096 else 48
            us = _time_calls(ctx, calls, iters, warm=4)
            nbytes = 2 * one + 2 * n_heads * hd * 4
            row = {"context": L, "us_per_call": round(us, 2), "GB/s": round(nbytes / us / 1e3, 1),
                   "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                   "rotating_caches": n_rot, "working_set_MB": round(2 * one * n_rot / 1e6, 1),
                   "hbm_streamed": 2 * one * n_rot > (256 << 20)}
            if tag:
                row["kv"] = tag
            if 2 * one <= 256 << 20 and n_rot > 1:
                us1 = _time_calls(ctx, calls[:1], iters, warm=4)
                row["one_cache_back_to_back_GB/s"] = round(nbytes / us1 / 1e3, 1)
            out.append(row)

    rows(ctx.lib.cera_hip_attn_decode_dev, 4, (512, 4096, 32768, 131072), None)
    # the same contexts over an f16 KV cache (KvCompression::F16): half the bytes per position
    chunk16 = chunk.astype(np.float16)
    dchunk16 = ctx.to_device(chunk16.view(np.uint16))
    for off in range(0, kv_bytes, chunk16.nbytes):
        ctx.check(ctx.lib.cera_hip_copy_dev(ctx.h, dk + off, dchunk16, chunk16.nbytes))
        ctx.check(ctx.lib.cera_hip_copy_dev(ctx.h, dv + off, dchunk16, chunk16.nbytes))
    rows(ctx.lib.cera_hip_attn_decode_f16_dev, 2, (4096, 32768, 131072), "f16")
    for d in (dk, dv, dchunk, dchunk16, dq, dout):
        ctx.free(d)
    return out


def measure_gemm(ctx, H, dts, shape, rng, n_thr=16):
    """BASELINE.json configs[2]: prefill GEMM out[N][M] = W_q . Q8_0(X[M][K]) on the matrix cores, activation
    quantization included in the timed call.  One extra row set, outside BASELINE: the gate shape in Q5_K, whose
    batched kernel reads the f32 activations (as the reference's Q5_K dot does) as split f16 operands."""
    INT8_PEAK_TOPS = 5000.0  # MI355X published dense int8 MFMA rate
    F16_PEAK_TOPS = 2500.0   # ... and dense f16
    res = []
    shape = dict(shape)
    dts = dict(dts)
    _, n_gate, k_gate = shape["ffn_gate"]
    w5 = rng.standard_normal((n_gate, k_gate), dtype=np.float32) * np.float32(0.02)
    dts["ffn_gate_q5_k"] = [ctx.tensor_upload(H.TYPE_IDS["Q5_K"], n_gate, k_gate, H.quantize(H.TYPE_IDS["Q5_K"], w5, n_thr))]
    shape["ffn_gate_q5_k"] = ("Q5_K", n_gate, k_gate)
    del w5
    for name in ("ffn_gate", "ffn_down", "ffn_gate_q5_k"):
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
            # Q4_K runs on the fp8 matrix cores (exact small-integer operands), the other 4-/8-bit types on int8: both 5.0 P(FL)OP/s dense
            peak_key, peak = (("frac_of_f16_mfma_peak", F16_PEAK_TOPS) if tname in ("Q6_K", "Q5_K") else
                              ("frac_of_fp8_mfma_peak", INT8_PEAK_TOPS) if tname == "Q4_K" else ("frac_of_int8_mfma_peak", INT8_PEAK_TOPS))
            res.append({"weight": f"{name} {tname} {n_out}x{k}", "tokens": m_tok, "us_per_call": round(us, 1),
                        "TOP/s": round(tops, 1), peak_key: round(tops / peak, 4)})
            ctx.free(dx)
            ctx.free(dout)
    ctx.tensor_free(dts["ffn_gate_q5_k"][0])
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
    for n_tok in (1, 2, 4, 8, 16, 32):
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


def reference_decode_threads(physical, logical):
    """The decode pool width cera picks for a bandwidth-bound model (more than 2.5 MB of weights per pool
    dispatch, which an 8B model is): physical + physical / 4 capped at 24, never above the detected
    logical count (cera README.md "How the decode thread count is chosen", CERA_DECODE_WIDE)."""
    if not physical:
        return max(1, min(12, logical or 1))   # the flat cap the sizing falls back to
    return max(1, min(24, physical + physical // 4, logical or physical))


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--seed", type=int, default=20250)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--cpu-threads", type=int, default=0,
                    help="CPU-baseline pool width (default: the reference's own decode sizing rule for this host, "
                         "capped at the 16 cores a one-GPU box gives a job)")
    ap.add_argument("--weight-copies", type=int, default=N_LAYERS,
                    help="distinct HBM copies of the layer weights the step rotates over (default: one per layer; "
                         "fewer lets the last-level cache hold them, which is NOT the reported configuration)")
    ap.add_argument("--no-e2e", action="store_true", help="skip the end-to-end model run (prefill 512 + greedy 256)")
    ap.add_argument("--no-extras", action="store_true", help="skip the flash-decode and prefill-GEMM side measurements")
    ap.add_argument("--roofline-probe", action="store_true",
                    help="run only what roofline.avg_launch_us is taken from: the back-to-back launches of the fused "
                         "gate|up kernel over the rotating layer copies, HIP events around them; prints that figure as "
                         "JSON (the command whose rocprofv3 kernel trace is committed next to it)")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="run only a 1 GiB copy kernel, a few launches of each per-layer GEMV kernel, decode attention at "
                         "131072 and 8192 keys and the two prefill GEMMs at 2048 tokens, for a hardware-counter pass under "
                         "rocprofv3 --pmc; prints no JSON")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the hot path has no multi-GPU part); "
              "run with --gpus 1", file=sys.stderr)
        return 2

    from cera_amd import hip_api, host_api as H
    Op = hip_api.DecodeOp

    ctx = hip_api.Context(0)
    dev_name, n_cu, hbm = ctx.device_info()
    rng = np.random.default_rng(args.seed)
    n_thr = min(16, os.cpu_count() or 1)
    eps = 1e-5

    # ---- synthetic weights: one properly quantized layer + head, cloned on device
    t0 = time.time()
    host = {}
    for name, tname, m, k in LAYER_SET + [HEAD] + [CONFIG1]:
        w = rng.standard_normal((m, k), dtype=np.float32)
        w *= np.float32(0.02)
        host[name] = H.quantize(H.TYPE_IDS[tname], w, n_thr)
        del w
    n_copies = max(1, min(N_LAYERS, args.weight_copies))
    dts = {}   # name -> list of device tensor handles (one per layer)
    for name, tname, m, k in LAYER_SET + [CONFIG1]:
        first = ctx.tensor_upload(H.TYPE_IDS[tname], m, k, host[name])
        copies = [first] + [ctx.tensor_clone(first) for _ in range(n_copies - 1)]
        dts[name] = [copies[l % len(copies)] for l in range(N_LAYERS)]
    name, tname, m, k = HEAD
    dts[name] = [ctx.tensor_upload(H.TYPE_IDS[tname], m, k, host[name])]
    gen_s = time.time() - t0

    # ---- inputs resident before timing: the f32 hidden state and norm weight the fused launches
    # read, and Q8_0-quantized activations for the projections whose input arrives quantized
    x_host = {kk: rng.standard_normal(kk, dtype=np.float32) for kk in (4096, 14336)}
    norm_host = (1.0 + 0.1 * rng.standard_normal(4096)).astype(np.float32)
    d_x = {kk: ctx.to_device(x_host[kk]) for kk in x_host}
    d_norm = ctx.to_device(norm_host)
    acts = {}
    for kk in (4096, 14336):
        dxs, dxq = ctx.malloc(kk // 32 * 4), ctx.malloc(kk)
        ctx.check(ctx.lib.cera_hip_quantize_q8_0_dev(ctx.h, d_x[kk], kk, dxs, dxq))
        acts[kk] = (dxs, dxq)
    outs = {name: ctx.malloc(m * 4) for name, _, m, _ in LAYER_SET + [HEAD] + [CONFIG1]}
    d_ffn_q, d_ffn_s = ctx.malloc(14336), ctx.malloc(14336 // 32 * 4)     # the gate|up launch's Q8_0 output
    d_head_in = ctx.malloc(4096 * 4)
    d_head_q, d_head_s = ctx.malloc(4096), ctx.malloc(4096 // 32 * 4)
    d_oq, d_os = ctx.malloc(4096), ctx.malloc(4096 // 32 * 4)
    ctx.sync()

    def op_qkv(l, t=None):
        return Op(kind=Op.NORM_GEMV, w=(t or dts)["attn_qkv"][l], x=d_x[4096], norm_w=d_norm, eps=eps, y=outs["attn_qkv"])

    def op_o(l, xs=None, xq=None, t=None):
        return Op(kind=Op.GEMV, w=(t or dts)["attn_output"][l], xs=xs or acts[4096][0], xq=xq or acts[4096][1], resid=d_x[4096],
                  y=outs["attn_output"])

    def op_gate_up(l, t=None):
        return Op(kind=Op.NORM_GATE_UP, w=(t or dts)["ffn_gate"][l], w2=(t or dts)["ffn_up"][l], x=d_x[4096], norm_w=d_norm, eps=eps,
                  out_q=d_ffn_q, out_s=d_ffn_s)

    def op_down(l, fused_input=True, t=None):
        xs, xq = (d_ffn_s, d_ffn_q) if fused_input else acts[14336]
        return Op(kind=Op.GEMV, w=(t or dts)["ffn_down"][l], xs=xs, xq=xq, resid=d_x[4096], y=outs["ffn_down"])

    op_head_norm = Op(kind=Op.NORM_QUANT, n=4096, x=d_x[4096], norm_w=d_norm, eps=eps, y=d_head_in, out_q=d_head_q, out_s=d_head_s)
    op_head = Op(kind=Op.GEMV, w=dts["output"][0], xs=d_head_s, xq=d_head_q, y=outs["output"])
    op_quant_o = Op(kind=Op.QUANT, n=4096, x=d_x[4096], out_q=d_oq, out_s=d_os)

    def ops_array(ops):
        arr = (Op * len(ops))()
        for i, o in enumerate(ops):
            arr[i] = o
        return arr

    # one token: the decode path's launches in its order (attention itself is not part of the set)
    step_ops = []
    for l in range(N_LAYERS):
        step_ops += [op_qkv(l), op_o(l), op_gate_up(l), op_down(l)]
    step_ops += [op_head_norm, op_head]
    step_arr = ops_array(step_ops)
    # the same with the one quantization the decode path gets from its attention kernel done as a
    # launch of its own: every Q8_0 quantization the reference performs per GEMV call is then inside
    step_q_ops = []
    for l in range(N_LAYERS):
        step_q_ops += [op_qkv(l), op_quant_o, op_o(l, d_os, d_oq), op_gate_up(l), op_down(l)]
    step_q_ops += [op_head_norm, op_head]
    step_q_arr = ops_array(step_q_ops)

    shape = {n: (t, m, k) for n, t, m, k in LAYER_SET + [HEAD] + [CONFIG1]}
    wbytes = {n: shape[n][1] * H.row_bytes(H.TYPE_IDS[shape[n][0]], shape[n][2]) for n in shape}
    # algorithmic bytes per launch: weights once, every input and output vector once
    launch_bytes = {
        "attn_qkv": wbytes["attn_qkv"] + 2 * 4096 * 4 + 6144 * 4,
        "attn_output": wbytes["attn_output"] + 4096 + 4096 // 32 * 4 + 2 * 4096 * 4,
        "ffn_gate_up": wbytes["ffn_gate"] + wbytes["ffn_up"] + 2 * 4096 * 4 + 14336 + 14336 // 32 * 4,
        "ffn_down": wbytes["ffn_down"] + 14336 + 14336 // 32 * 4 + 2 * 4096 * 4,
        "head_norm_quant": 3 * 4096 * 4 + 4096 + 4096 // 32 * 4,
        "output": wbytes["output"] + 4096 + 4096 // 32 * 4 + 128256 * 4,
        "config1_q4_0": algorithmic_bytes(H, *shape["config1_q4_0"]),
    }
    step_bytes = N_LAYERS * sum(launch_bytes[n] for n in ("attn_qkv", "attn_output", "ffn_gate_up", "ffn_down")) \
        + launch_bytes["head_norm_quant"] + launch_bytes["output"]
    weight_bytes = sum(N_LAYERS * len(host[n]) for n, *_ in LAYER_SET) + len(host["output"])

    def run(arr):
        ctx.check(ctx.lib.cera_hip_decode_ops_dev(ctx.h, arr, len(arr)))

    # per-kernel groups: 32 back-to-back launches of one kind over the rotating layer copies
    groups = {
        "attn_qkv": ops_array([op_qkv(l) for l in range(N_LAYERS)]),
        "attn_output": ops_array([op_o(l) for l in range(N_LAYERS)]),
        "ffn_gate_up": ops_array([op_gate_up(l) for l in range(N_LAYERS)]),
        "ffn_down": ops_array([op_down(l, fused_input=False) for l in range(N_LAYERS)]),
        "output": ops_array([op_head]),
        "config1_q4_0": ops_array([Op(kind=Op.GEMV, w=dts["config1_q4_0"][l], xs=acts[4096][0], xq=acts[4096][1],
                                      y=outs["config1_q4_0"]) for l in range(N_LAYERS)]),
    }

    if args.pmc_probe:
        n = 1 << 30
        src, dst = ctx.malloc(n), ctx.malloc(n)
        ctx.check(ctx.lib.cera_hip_copy_kernel(ctx.h, dst, src, n))   # first touch
        for _ in range(3):
            ctx.check(ctx.lib.cera_hip_copy_kernel(ctx.h, dst, src, n))
        for _ in range(2):
            for g in ("ffn_gate_up", "ffn_down", "attn_qkv", "attn_output"):
                run(groups[g])
        # decode attention, 32/8/128 heads, f32 cache (the values do not matter to the counters): 131072 keys take
        # one wavefront per head group and non-temporal reads, 8192 and 9216 keys two wavefronts per group and
        # cached reads (9216 keys make 15 workgroups per kv head and sub-group, not a multiple of the 8 XCDs)
        import ctypes as C
        kv_b = 8 * 131072 * 128 * 4
        dkp, dvp = ctx.malloc(kv_b), ctx.malloc(kv_b)
        dqp, dop = ctx.to_device(rng.standard_normal(32 * 128, dtype=np.float32)), ctx.malloc(32 * 128 * 4)
        for L in (131072, 8192, 9216):
            for _ in range(4):
                ctx.check(ctx.lib.cera_hip_attn_decode_dev(ctx.h, dqp, dkp, dvp, 32, 8, 128, L, L, C.c_float(1.0 / np.sqrt(128.0)), 0, dop))
        ctx.sync()
        for d in (dkp, dvp, dqp, dop):
            ctx.free(d)
        # the prefill GEMMs at 2048 tokens: Q4_K gate (int8 matrix core) and Q6_K down (f16 matrix core)
        m_tok = 2048
        for name in ("ffn_gate", "ffn_down"):
            _, n_out, kk = shape[name]
            dxg = ctx.to_device(rng.standard_normal((m_tok, kk), dtype=np.float32))
            dog = ctx.malloc(n_out * m_tok * 4)
            for _ in range(3):
                ctx.check(ctx.lib.cera_hip_gemm_dev(ctx.h, dts[name][0], dxg, m_tok, dog))
            ctx.sync()
            ctx.free(dxg)
            ctx.free(dog)
        ctx.sync()
        print(f"pmc probe done: copy kernel {n} B read + {n} B written per launch; algorithmic B per launch: "
              + ", ".join(f"{g} {launch_bytes[g]}" for g in ("ffn_gate_up", "ffn_down", "attn_qkv", "attn_output")),
              file=sys.stderr)
        return 0

    # set-up, whatever --warmup says: a matrix's first use builds its decode copy (an allocation and a
    # permutation kernel per matrix), which belongs to loading the weights, not to a step
    run(step_arr)
    ctx.sync()

    ROOFLINE_REPS = 8

    def time_group(arr, reps):
        """HIP events on the launch stream around reps back-to-back passes over arr: us per launch."""
        for _ in range(2):
            run(arr)
        e0, e1 = ctx.event(), ctx.event()
        ctx.record(e0)
        for _ in range(reps):
            run(arr)
        ctx.record(e1)
        ctx.sync()
        return ctx.elapsed_ms(e0, e1) * 1e3 / (reps * len(arr))

    if args.roofline_probe:
        us = time_group(groups["ffn_gate_up"], ROOFLINE_REPS)
        print(json.dumps({"kernel": GATE_UP_KERNEL, "launches": (ROOFLINE_REPS + 2) * N_LAYERS + N_LAYERS,
                          "avg_launch_us_hip_events": round(us, 3), "bytes_per_launch": launch_bytes["ffn_gate_up"],
                          "GB/s": round(launch_bytes["ffn_gate_up"] / us / 1e3, 1),
                          "frac": round(launch_bytes["ffn_gate_up"] / us / 1e3 / HBM_PEAK_GBS, 4)}))
        return 0
    for _ in range(args.warmup):
        run(step_arr)
    ctx.sync()

    # ---- timed region: exactly --steps steps, bracketed by synchronisation; an event pair per step
    evs = [(ctx.event(), ctx.event()) for _ in range(args.steps)]
    ctx.sync()
    t_start = time.perf_counter()
    for s in range(args.steps):
        ctx.record(evs[s][0])
        run(step_arr)
        ctx.record(evs[s][1])
    ctx.sync()
    wall = time.perf_counter() - t_start
    step_ms = sorted(ctx.elapsed_ms(a, b) for a, b in evs)
    ms_per_step = wall * 1e3 / args.steps
    value = step_bytes / (wall / args.steps) / 1e9
    p50 = step_ms[len(step_ms) // 2]
    p10, p90 = step_ms[len(step_ms) // 10], step_ms[min(len(step_ms) - 1, len(step_ms) * 9 // 10)]

    # ---- the set with every per-call Q8_0 quantization of the reference inside (cpu.rs:787-790)
    q_steps = max(10, args.steps // 2)
    for _ in range(2):
        run(step_q_arr)
    ctx.sync()
    t_q = time.perf_counter()
    for _ in range(q_steps):
        run(step_q_arr)
    ctx.sync()
    ms_q = (time.perf_counter() - t_q) * 1e3 / q_steps
    bytes_q = step_bytes + N_LAYERS * (4096 * 4 + 4096 + 4096 // 32 * 4)

    # ---- per matrix: HIP events around 32 back-to-back launches of one kernel, rotating copies
    per_matrix = {}
    reps = ROOFLINE_REPS
    for g, arr in groups.items():
        us = time_group(arr, reps * (8 if len(arr) == 1 else 1))
        tname, m, k = shape["ffn_gate" if g == "ffn_gate_up" else g]
        per_matrix[g] = {"weights": ("2 x " if g == "ffn_gate_up" else "") + f"{tname} {m}x{k}", "us_per_launch": round(us, 2),
                         "bytes_per_launch": launch_bytes[g], "GB/s": round(launch_bytes[g] / us / 1e3, 1),
                         "frac_of_hbm_peak": round(launch_bytes[g] / us / 1e3 / HBM_PEAK_GBS, 4),
                         "cache_resident": len(arr) == 1 and False}
    per_matrix["output"]["note"] = "one 431 MB matrix launched back to back: larger than the 256 MB last-level cache"
    for g in per_matrix:
        per_matrix[g].pop("cache_resident")

    # dominant kernel: the fused Q4_K gate|up launch, 2 x (14336 x 4096) per launch, 32 launches per step
    gu = per_matrix["ffn_gate_up"]
    roofline = {"bound": "hbm", "kernel": GATE_UP_KERNEL + " (rmsnorm + Q8_0 in, Q4_K gate | up 2 x 14336x4096, SwiGLU + Q8_0 out)",
                "achieved": gu["GB/s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(gu["GB/s"] / HBM_PEAK_GBS, 4), "traffic": GATE_UP_TRAFFIC_BYTES,
                "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE passes over bench.py --pmc-probe, "
                                  "calibrated on a 1 GiB copy kernel (recorded, see profiles/)",
                "bytes_per_launch": launch_bytes["ffn_gate_up"], "avg_launch_us": gu["us_per_launch"],
                "avg_launch_source": f"HIP events on the launch stream around {reps} x 32 back-to-back launches over "
                                     f"{n_copies} rotating layer copies, taken right after the timed region; "
                                     "`bench.py --roofline-probe` runs exactly this loop, and its rocprofv3 kernel trace is "
                                     "profiles/gemv_gate_up_back_to_back_kernel_trace.txt",
                "trace_avg_launch_us_back_to_back": GATE_UP_TRACE_BACK_TO_BACK_US,
                "frac_at_trace_avg_back_to_back": round(launch_bytes["ffn_gate_up"] / GATE_UP_TRACE_BACK_TO_BACK_US / 1e3 / HBM_PEAK_GBS, 4),
                "avg_launch_us_in_decode_step": GATE_UP_IN_STEP_US,
                "frac_in_decode_step": round(launch_bytes["ffn_gate_up"] / GATE_UP_IN_STEP_US / 1e3 / HBM_PEAK_GBS, 4),
                "in_decode_step_source": "rocprofv3 --kernel-trace --stats over the whole default bench.py run "
                                         "(recorded, profiles/gemv_decode_set_llama3_8b_kernel_trace.txt): between the other "
                                         "kernels of a step the same launch averages longer than back to back"}

    # ---- the same step on the native GGUF layout: decode copies off, freshly uploaded tensors
    ctx.set_decode_copies(False)
    try:
        nat = {}
        for name, tname, m, k in LAYER_SET:
            first = ctx.tensor_upload(H.TYPE_IDS[tname], m, k, host[name])
            copies = [first] + [ctx.tensor_clone(first) for _ in range(n_copies - 1)]
            nat[name] = [copies[l % len(copies)] for l in range(N_LAYERS)]
        name, tname, m, k = HEAD
        nat_head = ctx.tensor_upload(H.TYPE_IDS[tname], m, k, host[name])
        nat_ops = []
        for l in range(N_LAYERS):
            nat_ops += [op_qkv(l, nat), op_o(l, t=nat), op_gate_up(l, nat), op_down(l, t=nat)]
        nat_ops += [op_head_norm, Op(kind=Op.GEMV, w=nat_head, xs=d_head_s, xq=d_head_q, y=outs["output"])]
        nat_arr = ops_array(nat_ops)
        for _ in range(max(2, args.warmup)):
            run(nat_arr)
        ctx.sync()
        t_n = time.perf_counter()
        for _ in range(args.steps):
            run(nat_arr)
        ctx.sync()
        native_gbs = step_bytes / ((time.perf_counter() - t_n) / args.steps) / 1e9
        for lst in nat.values():
            for t in {id(x): x for x in lst}.values():
                ctx.tensor_free(t)
        ctx.tensor_free(nat_head)
    finally:
        ctx.set_decode_copies(True)

    # ---- correctness spot check of what was just timed (oracle is only the checker)
    cpu_baseline = None
    if not args.no_cpu_baseline:
        from oracle import binding as orc
        name = "attn_output"
        tname, m, k = shape[name]
        y = ctx.download(outs[name], (m,), np.float32)
        ref = x_host[4096] + orc.gemv(H.TYPE_IDS[tname], host[name], x_host[k], m, k)
        rel = float(np.abs(y - ref).max() / np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
        assert rel <= 1e-3, f"GPU result of the timed GEMV deviates from the oracle: {rel}"
        fq = ctx.download(d_ffn_q, (14336,), np.int8)
        normed = orc.rmsnorm(x_host[4096], norm_host, eps)
        act = orc.silu_mul(orc.gemv(H.TYPE_IDS["Q4_K"], host["ffn_gate"], normed, 14336, 4096),
                           orc.gemv(H.TYPE_IDS["Q4_K"], host["ffn_up"], normed, 14336, 4096))
        _, want_q = orc.quantize_q8_0(act)
        off = np.abs(fq.astype(np.int32) - want_q.astype(np.int32))
        assert off.max() <= 1 and np.count_nonzero(off) <= 14336 // 50, "fused gate|up output deviates from the oracle"
        # CPU baseline: the restated cera AVX2 int8 path on a bounded sample --
        # whole layers' GEMV sets (QKV, O, gate, up, down), rotating over distinct
        # weight copies so the host LLC does not hold them.
        info = host_cpu_info()
        policy = reference_decode_threads(info["physical_cores"], info["logical_cores"])
        cpu_thr = args.cpu_threads or max(1, min(policy, 16))
        pool = orc.Pool(cpu_thr)
        n_cp = 8
        layer_sets = []
        for c in range(n_cp):
            layer_sets.append({n: (host[n] if c == 0 else host[n].copy()) for n, *_ in LAYER_SET})
        ybuf = {n: np.empty(shape[n][1], np.float32) for n, *_ in LAYER_SET}
        layer_bytes = sum(algorithmic_bytes(H, *shape[n]) for n, *_ in LAYER_SET)
        done_layers = 0
        t_cpu = time.perf_counter()
        while time.perf_counter() - t_cpu < args.cpu_seconds or done_layers < 2:
            ws = layer_sets[done_layers % n_cp]
            for n, tname, m, k in LAYER_SET:
                pool.gemv(H.TYPE_IDS[tname], ws[n], x_host[k], m, k, ybuf[n])
            done_layers += 1
        cpu_s = time.perf_counter() - t_cpu
        pool.close()
        cpu_baseline = {"value": round(done_layers * layer_bytes / cpu_s / 1e9, 2), "unit": "GB/s",
                        "cores": cpu_thr, "kind": "port",
                        "sample": f"{done_layers} decode-layer GEMV sets (QKV, O, gate, up Q4_K; down Q6_K; "
                                  f"{layer_bytes} B each) in {cpu_s:.1f} s, restated cera AVX2 int8 path "
                                  f"incl. per-call Q8_0 quantize, {n_cp} rotating weight copies",
                        "threads_policy": f"cera's decode sizing for a bandwidth-bound model: physical + physical/4 <= 24 "
                                          f"= {policy} on this host, capped at the 16 cores of a one-GPU job",
                        "avx2": bool(orc.lib().orc_have_avx2()), **info}

    extras = {}
    if not args.no_extras:
        extras["flash_decode"] = measure_attention(ctx, hip_api, rng)
        extras["prefill_gemm"] = measure_gemm(ctx, H, dts, shape, rng, n_thr)
    e2e = None if args.no_e2e else measure_e2e(args.seed, n_thr)
    # the metric names tok/s too: the end-to-end rates ride in `config`, next to the workload they belong to
    e2e_cfg = None if e2e is None else {
        "workload": "random-init Llama-3-8B arch GGUF (Q4_K_M-style mix) through HipLlamaModel: prefill 512 + greedy 256, batch 1",
        "decode_tok_s": e2e["decode_tok_s"], "prefill_tok_s": e2e["prefill_tok_s"],
        "decode_frac_of_hbm_peak": e2e["decode_frac_of_hbm_peak"]}

    out = {
        "metric": "Q4_K GEMV HBM GB/s (% of peak); Llama-3-8B-arch Q4_K decode tok/s, 1 GPU",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": "Llama-3-8B decode-layer GEMV set, batch 1, decode order: 32 x (QKV 6144x4096 with rmsnorm+Q8_0 "
                               "inside, O 4096x4096, gate|up 2 x 14336x4096 Q4_K with rmsnorm+Q8_0 in and SwiGLU+Q8_0 out; "
                               "down 4096x14336 Q6_K) + rmsnorm+Q8_0 + head 128256x4096 Q6_K",
                   "launches_per_step": len(step_ops), "weight_bytes_per_step": weight_bytes,
                   "algorithmic_bytes_per_step": step_bytes, "w_sigma": 0.02, "seed": args.seed,
                   "distinct_weight_copies": n_copies,
                   "weight_layout": "each matrix read from its decode copy (per-row permutation of the GGUF bytes, the "
                                    "library's default, built before the timed region); same bytes per step",
                   "native_layout_GB/s": round(native_gbs, 1),
                   "native_layout": "the same step with decode copies off: every matrix read from its GGUF bytes as uploaded",
                   "e2e": e2e_cfg},
        "native_layout_GB/s": round(native_gbs, 1),
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
        "ms_per_step_p50": round(p50, 4), "ms_per_step_p10": round(p10, 4), "ms_per_step_p90": round(p90, 4),
        "value_p50_GB/s": round(step_bytes / (p50 * 1e-3) / 1e9, 1),
        "set_incl_quantize_GB/s": round(bytes_q / (ms_q * 1e-3) / 1e9, 1),
        "set_incl_quantize": {"ms_per_step": round(ms_q, 4), "steps": q_steps, "launches_per_step": len(step_q_ops),
                              "what": "the same step with O's input quantized by a launch of its own: all five per-layer "
                                      "Q8_0 quantizations and the head's, which the reference performs per GEMV call, "
                                      "are inside the timed step (the decode path gets O's from its attention kernel)"},
        "gemv_only_tok_s_equiv": round(1e3 / ms_per_step, 1),
        "per_matrix": per_matrix,
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
