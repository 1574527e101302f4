"""Full-size end-to-end parity: a seeded random-init Llama-3-8B-architecture GGUF
(32 layers, d_model 4096, 32/8 GQA heads, ffn 14336, vocab 128256; Q4_K_M-style
mix), 512-token prefill of uniform random ids, then 256 greedy tokens -- the GPU
backend through HipLlamaModel against the CPU oracle on the same file.

The oracle side takes a few minutes of CPU time (and the file is 5.2 GB), so
the full test only runs when CERA_E2E_8B=1; a smaller number of layers can be chosen
with CERA_E2E_LAYERS for a quicker pass over the same per-layer shapes.  A cut of the
same architecture (4 layers, the full-width embedding and head, 128-token prefill,
32 greedy tokens; 1.4 GB, seconds of CPU time) runs with every GPU test run.
"""
import os
import time

import numpy as np
import pytest

import util
from cera_amd import host_api as H, llama_api, synth

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)


@pytest.mark.skipif(os.environ.get("CERA_E2E_8B") != "1", reason="set CERA_E2E_8B=1 (minutes of CPU time)")
def test_llama3_8b_prefill_512_greedy_256(tmp_path, orc, hip):
    n_layers = int(os.environ.get("CERA_E2E_LAYERS", synth.LLAMA3_8B["n_layers"]))
    _run(tmp_path, orc, n_layers, 512, int(os.environ.get("CERA_E2E_NEW", 256)))


def test_llama3_8b_shapes_4_layers_prefill_128_greedy_32(tmp_path, orc, hip):
    _run(tmp_path, orc, 4, 128, 32)


def _run(tmp_path, orc, n_layers, n_prompt, n_new):
    cfg = dict(synth.LLAMA3_8B, max_seq_len=1024)
    cfg["n_layers"] = n_layers
    threads = min(16, os.cpu_count() or 1)
    path = str(tmp_path / "llama3_8b_synth.gguf")
    t0 = time.time()
    H.synth_llama_gguf(path, cfg, seed=20240, n_threads=threads, explicit_head_dim=False)
    _say(f"e2e: wrote {os.path.getsize(path) / 1e9:.2f} GB in {time.time() - t0:.0f} s")
    prompt = util.rng(99).integers(0, cfg["vocab"], n_prompt).astype(np.uint32)

    gm = llama_api.HipLlama(path, context_size=1024)
    _say(f"e2e: model in HBM, {gm.gpu_memory_bytes / 1e9:.2f} GB")
    # free-running greedy decode, the workload as a user runs it
    toks, tp, td = gm.generate_greedy(prompt, n_new, ubatch=512)
    _say(f"e2e: GPU prefill {n_prompt / tp:.0f} tok/s, decode {(n_new - 1) / td:.1f} tok/s")
    # the same again step by step, keeping every step's logits
    gm.truncate_kv(0)
    g_logits = [gm.forward_prefill(prompt, 0)]
    for i in range(n_new - 1):
        g_logits.append(gm.forward(int(toks[i]), n_prompt + i))
    assert [int(np.argmax(l)) for l in g_logits] == [int(t) for t in toks], "GPU run is not reproducible"
    gm.close()

    rcfg, weights = H.Gguf(path).llama_weights()
    rcfg["max_seq_len"] = 1024
    pool = orc.Pool(threads)
    # Two oracle instances: A prefills through the batched GEMM route (what the reference runs
    # for n > 1), B through the per-token GEMV route.  They are the same algorithm up to how the
    # K-quant partial sums are split over accumulators, so |B - A| is the distance the reference
    # keeps from itself -- the floor any other implementation is measured against.
    oa, ob = orc.Llama(rcfg, weights), orc.Llama(rcfg, weights)
    oa.set_pool(pool); ob.set_pool(pool)
    t0 = time.time()
    la = oa.forward_prefill_batched(prompt, 0)
    _say(f"e2e: oracle batched prefill {time.time() - t0:.0f} s on {threads} threads")
    t0 = time.time()
    lb = ob.forward_prefill_per_token(prompt, 0)
    _say(f"e2e: oracle per-token prefill {time.time() - t0:.0f} s")

    def cos(x, y):
        x, y = x.astype(np.float64), y.astype(np.float64)
        return float(x @ y / np.sqrt((x @ x) * (y @ y)))

    def gap_rel(logits, a, b):   # cera/tests/gpu_transformer_parity.rs:207-212
        p, q = float(logits[a]), float(logits[b])
        return abs(p - q) / max(abs(p), abs(q), 1.0)

    same_g = same_b = 0
    worst_g = worst_b = 0.0   # largest margin of a disagreement, in units of the per-logit noise rms
    rel_g, rel_b, cos_g, cos_b = [], [], [], []
    t0 = time.time()
    for i in range(n_new):
        lg = g_logits[i]
        rel_g.append(util.rms(lg - la) / util.rms(la)); rel_b.append(util.rms(lb - la) / util.rms(la))
        cos_g.append(cos(lg, la)); cos_b.append(cos(lb, la))
        tg, ta, tb = int(toks[i]), int(orc.argmax(la)), int(orc.argmax(lb))
        same_b += ta == tb
        if ta != tb:
            worst_b = max(worst_b, max(float(la[ta] - la[tb]), float(lb[tb] - lb[ta])) / util.rms(lb - la))
        if ta == tg:
            same_g += 1
        else:
            # a disagreement must be explained by the measured logit noise on both sides: the
            # difference of two logits carries sqrt(2) x the per-logit noise, and with ~1e5
            # candidates x 256 steps a 4-sigma swing of some pair is expected, so the bound is
            # 5 sigma of the pair difference (7 x the per-logit rms)
            noise = util.rms(lg - la)
            m_a, m_g = float(la[ta] - la[tg]), float(lg[tg] - lg[ta])
            _say(f"  step {i}: GPU {tg} vs oracle {ta}: margins {m_a:.3f} / {m_g:.3f}, logit noise rms {noise:.3f}, "
                 f"relative gaps {gap_rel(la, ta, tg):.4f} / {gap_rel(lg, ta, tg):.4f}")
            worst_g = max(worst_g, max(m_a, m_g) / noise)
            assert m_a <= 7 * noise and m_g <= 7 * noise, f"step {i}: different token beyond the noise"
        if i + 1 < n_new:       # teacher-forced on the GPU's sequence
            la, lb = oa.forward(tg, n_prompt + i), ob.forward(tg, n_prompt + i)
    _say(f"e2e: oracle decode {time.time() - t0:.0f} s")
    _say(f"e2e: GPU vs oracle(batched):            identical greedy tokens {same_g}/{n_new}, "
         f"cosine min {min(cos_g):.5f} mean {np.mean(cos_g):.5f}, rms(diff)/rms mean {np.mean(rel_g):.4f}, "
         f"largest disagreement margin {worst_g:.1f} x noise")
    _say(f"e2e: oracle(per-token) vs oracle(batched): identical greedy tokens {same_b}/{n_new}, "
         f"cosine min {min(cos_b):.5f} mean {np.mean(cos_b):.5f}, rms(diff)/rms mean {np.mean(rel_b):.4f}, "
         f"largest disagreement margin {worst_b:.1f} x noise")
    oa.set_pool(None); ob.set_pool(None)
    pool.close()
    oa.close(); ob.close()
    # 0.99 is the floor the reference sets for its own flash-route (n >= 256) prefill comparison
    # (cera/tests/llama_batched_prefill_parity.rs:337-358)
    assert min(cos_g) >= 0.99
    # the GPU is no further from the oracle than the oracle's two routes are from each other
    assert np.mean(rel_g) <= 1.25 * np.mean(rel_b) + 1e-3
    assert n_new - same_g <= 1.5 * (n_new - same_b) + 4
