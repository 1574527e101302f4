"""GPU parity of the Model-trait layer: a GGUF file on disk -> HipLlamaModel
(C++ host layer over the C-ABI) against the oracle's LlamaModel twin built from
the very same file.  Mirrors the harness shape of the reference's test for a
new GPU backend (cera/tests/gpu_transformer_parity.rs:75-103: prefill, then
greedy continuation, logits compared per step with near-tie tolerance)."""
import json
import subprocess

import numpy as np
import pytest

import util
from cera_amd import _build, host_api as H, llama_api, synth

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)


def _cos(a, b):
    a = a.astype(np.float64); b = b.astype(np.float64)
    return float(a @ b / np.sqrt((a @ a) * (b @ b)))


def _close(lg, lo, what):
    err = float(np.abs(lg - lo).max())
    _say(f"  {what}: max|err|={err:.3e} rms={util.rms(lo):.3e} cos={_cos(lg, lo):.8f}")
    assert _cos(lg, lo) > 0.999 and err <= 0.1 * util.rms(lo), what
    return err


def _teacher_forced(gm, om, orc, prompt, n_new, min_same):
    lg = gm.forward_prefill(prompt, 0)
    lo = om.forward_prefill_per_token(prompt, 0)
    same = 0
    for i in range(n_new):
        err = _close(lg, lo, f"step {i}")
        tg, to = int(orc.argmax(lg)), int(orc.argmax(lo))
        if tg == to:
            same += 1
        else:
            srt = np.sort(lo)
            assert float(srt[-1] - srt[-2]) <= 2 * err, f"step {i}: {tg} vs {to} beyond a near-tie"
        pos = len(prompt) + i
        lg, lo = gm.forward(to, pos), om.forward(to, pos)
    assert same >= min_same, same


@pytest.fixture(scope="module")
def tiny_llama(tmp_path_factory, orc, hip):
    path = str(tmp_path_factory.mktemp("gguf") / "tiny.gguf")
    H.synth_llama_gguf(path, dict(synth.TINY), seed=77, sigma=0.05, norm_jitter=0.1)
    cfg, weights = H.Gguf(path).llama_weights()
    gm = llama_api.HipLlama(path, context_size=64)
    om = orc.Llama(cfg, weights)
    yield path, cfg, gm, om
    gm.close()
    om.close()


def test_config_comes_from_the_file(tiny_llama):
    path, cfg, gm, om = tiny_llama
    c = gm.config
    assert (c["n_layers"], c["hidden_size"], c["intermediate_size"], c["n_heads"], c["n_kv_heads"], c["head_dim"],
            c["vocab_size"]) == (cfg["n_layers"], cfg["hidden"], cfg["ffn"], cfg["n_heads"], cfg["n_kv_heads"],
                                 cfg["head_dim"], cfg["vocab"])
    assert c["max_seq_len"] == 64 and c["rope_type"] == 1
    assert gm.gpu_memory_bytes > sum(w[3].size for w in H.Gguf(path).llama_weights()[1].values() if isinstance(w, tuple))


def test_forward_and_prefill_match_the_oracle(tiny_llama, orc):
    path, cfg, gm, om = tiny_llama
    gm.truncate_kv(0); om.truncate(0)
    _say("hip_llama: teacher-forced greedy from a GGUF")
    _teacher_forced(gm, om, orc, [5, 400, 31, 2, 77, 123, 9], 20, 17)
    assert gm.seq_len == om.seq_len == 27


def test_generate_greedy_equals_stepwise_calls(tiny_llama):
    path, cfg, gm, om = tiny_llama
    prompt = [9, 8, 7, 300, 12]
    gm.truncate_kv(0)
    toks, tp, td = gm.generate_greedy(prompt, 12, ubatch=512)
    assert gm.seq_len == len(prompt) + 11 and tp > 0 and td > 0
    gm.truncate_kv(0)
    logits = gm.forward_prefill(prompt, 0)
    step = [int(np.argmax(logits))]
    while len(step) < 12:
        step.append(gm.forward_greedy(step[-1], gm.seq_len))
    assert list(toks) == step


def test_chunked_prefill_and_cancel(tiny_llama):
    path, cfg, gm, om = tiny_llama
    tokens = [3, 1, 4, 1, 5, 9, 2, 6, 5, 35]
    gm.truncate_kv(0)
    whole = gm.forward_prefill(tokens, 0)
    gm.truncate_kv(0)
    consumed, chunked = gm.forward_prefill_chunked(tokens, 0, ubatch=4)
    assert consumed == 10 and gm.seq_len == 10
    _close(chunked, whole, "chunked vs whole")
    gm.truncate_kv(0)
    consumed, same = gm.forward_prefill_chunked(tokens, 0, ubatch=0)       # 0 = one chunk
    assert consumed == 10 and np.array_equal(same, whole)
    # a cancel raised before the call still advances by exactly one chunk (mod.rs:323-329)
    gm.truncate_kv(0)
    gm.set_cancel(True)
    consumed, part = gm.forward_prefill_chunked(tokens, 0, ubatch=4)
    gm.set_cancel(False)
    assert consumed == 4 and gm.seq_len == 4 and part is not None
    consumed, none = gm.forward_prefill_chunked([], 4, ubatch=4)
    assert consumed == 0 and none is None


def test_truncate_then_replay_is_bit_identical(tiny_llama):
    path, cfg, gm, om = tiny_llama
    gm.truncate_kv(0)
    gm.forward_prefill([1, 2, 3, 4, 5, 6], 0)
    a = gm.forward(50, 6)
    gm.truncate_kv(6)
    assert gm.seq_len == 6
    b = gm.forward(50, 6)
    assert np.array_equal(a, b)
    gm.truncate_kv(7)          # len == seq_len: the common, free case
    assert gm.seq_len == 7


def test_contract_violations_fail_loudly(tiny_llama):
    path, cfg, gm, om = tiny_llama
    gm.truncate_kv(0)
    gm.forward(1, 0)
    for call, needle in ((lambda: gm.forward(1, 5), "pos"), (lambda: gm.forward_prefill([1, 2], 3), "start_pos"),
                         (lambda: gm.forward(cfg["vocab"], 1), "out of range"),
                         (lambda: gm.truncate_kv(3), "exceeds"),
                         (lambda: gm.forward_prefill(list(range(70)), 1), "")):
        with pytest.raises(llama_api.BackendError) as e:
            call()
        assert needle in str(e.value), str(e.value)
    assert gm.seq_len == 1
    lg = gm.forward(2, 1)       # still usable after refused calls
    assert np.isfinite(lg).all()


def test_qwen3_style_file(tmp_path, orc, hip):
    """NEOX RoPE, Q/K/V biases, per-head QK-norm, tied output head, other weight types."""
    path = str(tmp_path / "q3.gguf")
    H.synth_llama_gguf(path, dict(synth.TINY), seed=5, sigma=0.05, norm_jitter=0.1, arch="qwen3", tied_output=True,
                       qkv_bias=True, qk_norm=True,
                       types=dict(token_embd=H.Q8_0, attn_q=H.Q4_0, attn_k=H.Q4_0, attn_v=H.Q4_0, attn_output=H.Q8_0,
                                  ffn_down=H.Q4_K))
    cfg, weights = H.Gguf(path).llama_weights()
    gm = llama_api.HipLlama(path, context_size=64)
    om = orc.Llama(cfg, weights)
    try:
        assert gm.config["rope_type"] == 0
        _say("hip_llama: qwen3-style file")
        _teacher_forced(gm, om, orc, [11, 22, 33, 44, 55], 12, 10)
    finally:
        gm.close(); om.close()


def test_context_size_caps_max_seq_len(tiny_llama):
    path = tiny_llama[0]
    gm = llama_api.HipLlama(path, context_size=8)
    try:
        assert gm.config["max_seq_len"] == 8
        gm.forward_prefill(list(range(8)), 0)
        with pytest.raises(llama_api.BackendError):
            gm.forward(1, 8)
    finally:
        gm.close()


def test_cli_run_agrees_with_the_library(tiny_llama):
    path, cfg, gm, om = tiny_llama
    _say("hip_llama: cera-hip run")
    r = subprocess.run([str(_build.CLI_BIN), "run", "--model", path, "--prompt-len", "12", "--n-predict", "6",
                        "--seed", "3", "--ctx", "64", "--tokens-out", path + ".tok"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    rep = json.loads(r.stdout.strip().splitlines()[-1])
    assert rep["prompt_len"] == 12 and rep["n_predict"] == 6 and rep["decode_tok_s"] > 0 and rep["prefill_tok_s"] > 0
    prompt, out = (list(map(int, line.split())) for line in open(path + ".tok").read().strip().splitlines())
    assert len(prompt) == 12 and len(out) == 6 and max(prompt) < cfg["vocab"]
    gm.truncate_kv(0)
    toks, _, _ = gm.generate_greedy(prompt, 6)
    assert list(toks) == out


def test_all_position_logits_match_per_token_forward(tiny_llama, orc, hip):
    """cera/tests/spec_decode_logits.rs:72-115: [n * vocab] rows, KV appended for all n tokens,
    every row against the per-token forward of the same position (cosine floor 0.99 there;
    the tighter 0.999 and a near-tie argmax here)."""
    path, cfg, gm, om = tiny_llama
    toks = [int(t) for t in util.rng(21).integers(0, cfg["vocab"], 24)]
    gm.truncate_kv(0); om.truncate(0)
    _say("hip_llama: all-position logits, 24 tokens")
    rows = gm.forward_prefill_logits_all(toks, 0)
    assert rows.shape == (24, cfg["vocab"]) and gm.seq_len == 24
    for i, t in enumerate(toks):
        lo = om.forward(t, i)
        err = _close(rows[i], lo, f"pos {i}")
        if int(orc.argmax(rows[i])) != int(orc.argmax(lo)):
            srt = np.sort(lo)
            assert float(srt[-1] - srt[-2]) <= 2 * err, i
    # the last row is what forward_prefill returns for the same prompt (GEMM vs GEMV head: float order only)
    gm.truncate_kv(0)
    last = gm.forward_prefill(toks, 0)
    assert np.abs(rows[-1] - last).max() <= 1e-3 * util.rms(last)
    # the cache it leaves continues like forward_prefill's
    om_next, gm_next = om.forward(7, 24), gm.forward(7, 24)
    _close(gm_next, om_next, "decode after prefill")
    # a second call on top of the cache (start_pos > 0), and the single-token form
    gm.truncate_kv(24); om.truncate(24)
    more = [3, 99, 250, 17, 8]
    rows2 = gm.forward_prefill_logits_all(more, 24)
    for i, t in enumerate(more):
        _close(rows2[i], om.forward(t, 24 + i), f"pos {24 + i}")
    one = gm.forward_prefill_logits_all([11], 29)
    _close(one[0], om.forward(11, 29), "single token")
    assert gm.seq_len == om.seq_len == 30
    with pytest.raises(llama_api.BackendError):
        gm.forward_prefill_logits_all([1, 2], 5)  # start_pos must equal the cache length
    with pytest.raises(llama_api.BackendError):
        gm.forward_prefill_logits_all([], 30)


def test_truncate_restores_the_cache(tiny_llama):
    """cera/tests/spec_decode_logits.rs:130-178: prefill 0..8, truncate to 4, prefill 4..8 gives
    the logits of prefill 0..4 then 4..8 (max |diff| < 1e-3 and the same argmax)."""
    path, cfg, gm, om = tiny_llama
    toks = [1, 150, 318, 297, 422, 298, 306, 62]
    gm.truncate_kv(0)
    gm.forward_prefill(toks[:4], 0)
    ref = gm.forward_prefill(toks[4:], 4)
    gm.truncate_kv(0)
    gm.forward_prefill(toks, 0)
    assert gm.seq_len == 8
    gm.truncate_kv(4)
    assert gm.seq_len == 4
    got = gm.forward_prefill(toks[4:], 4)
    assert gm.seq_len == 8
    assert int(np.argmax(ref)) == int(np.argmax(got)) and float(np.abs(ref - got).max()) < 1e-3


def test_shift_and_snapshot_through_the_model_layer(tiny_llama, tmp_path):
    """Model::shift_kv keeps the session's seq_len in step; snapshot_state / restore_state
    (cera/src/model/mod.rs:507-533) bring a second model to the same state: the next logits
    are bit-identical to the snapshotted model's."""
    path, cfg, gm, om = tiny_llama
    assert gm.supports_kv_shift
    toks = [int(t) for t in util.rng(41).integers(0, cfg["vocab"], 30)]
    gm.truncate_kv(0); om.truncate(0)
    gm.forward_prefill(toks, 0)
    om.forward_prefill_batched(toks, 0)
    snap = gm.snapshot_state()
    assert snap.seq_len == 30
    assert snap.nbytes == cfg["n_layers"] * 2 * 30 * cfg["n_kv_heads"] * cfg["head_dim"] * 4
    other = llama_api.HipLlama(path, context_size=64)
    other.restore_state(snap)
    assert other.seq_len == 30
    a, b = gm.forward(9, 30), other.forward(9, 30)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    # restoring rewinds: the snapshot predates token 9
    gm.restore_state(snap)
    assert gm.seq_len == 30
    c = gm.forward(9, 30)
    assert np.array_equal(a.view(np.uint32), c.view(np.uint32))
    other.close(); snap.close()
    # shift through the Model layer, against the oracle
    gm.truncate_kv(30); om.truncate(30)
    gm.shift_kv(2, 10); om.shift_kv(2, 10)
    assert gm.seq_len == om.seq_len == 20
    _close(gm.forward(5, 20), om.forward(5, 20), "after shift")
    with pytest.raises(llama_api.BackendError):
        gm.shift_kv(20, 5)
    with pytest.raises(llama_api.BackendError):
        gm.shift_kv(1, 0)
    assert gm.seq_len == 21


def test_f16_kv_through_the_model_layer(tiny_llama, orc):
    """f16_kv_supported + configure_kv_compression (cera/src/model/mod.rs:557-603), an f16
    snapshot at half the bytes, and the cross-mode restore gate (cera/src/kv_cache.rs:1411-1421)."""
    path, cfg, gm32, om32 = tiny_llama
    gm = llama_api.HipLlama(path, context_size=64)
    assert gm.f16_kv_supported
    gm.configure_kv_compression(True)
    with pytest.raises(llama_api.BackendError):
        gm.configure_kv_compression(False)
    _, weights = H.Gguf(path).llama_weights()
    om = orc.Llama(cfg, weights)
    om.set_kv_f16(True)
    toks = [int(t) for t in util.rng(61).integers(0, cfg["vocab"], 18)]
    _close(gm.forward_prefill(toks, 0), om.forward_prefill_batched(toks, 0), "f16 prefill")
    _close(gm.forward(4, 18), om.forward(4, 18), "f16 decode")
    snap = gm.snapshot_state()
    assert snap.seq_len == 19
    assert snap.nbytes == cfg["n_layers"] * 2 * 19 * cfg["n_kv_heads"] * cfg["head_dim"] * 2
    a = gm.forward(8, 19)
    gm.restore_state(snap)
    b = gm.forward(8, 19)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    gm32.truncate_kv(0)
    with pytest.raises(llama_api.BackendError):
        gm32.restore_state(snap)          # an f16 snapshot does not load into an f32 cache
    gm.close(); om.close(); snap.close()


@pytest.mark.parametrize("arch,explicit", [("llama", False), ("qwen3", True)])
def test_head_dim_64_file(tmp_path, orc, hip, arch, explicit):
    """Llama-3.2-1B / Granite-2B shape class: head_dim 64, implied by hidden / n_heads (llama) or
    given by attention.key_length and decoupled from it (qwen3: 8 heads x 64 over hidden 256)."""
    cfg0 = dict(synth.TINY, n_heads=8 if explicit else 4, n_kv_heads=2, head_dim=64)
    path = str(tmp_path / "hd64.gguf")
    H.synth_llama_gguf(path, cfg0, seed=15, sigma=0.05, norm_jitter=0.1, arch=arch, qk_norm=(arch == "qwen3"),
                       explicit_head_dim=explicit)
    cfg, weights = H.Gguf(path).llama_weights()
    assert cfg["head_dim"] == 64
    gm = llama_api.HipLlama(path, context_size=64)
    om = orc.Llama(cfg, weights)
    try:
        assert gm.config["head_dim"] == 64
        _say(f"hip_llama: head_dim 64 {arch} file")
        _teacher_forced(gm, om, orc, [11, 22, 33, 44, 55, 66, 77], 14, 12)
    finally:
        gm.close(); om.close()


# ---- a speculative-decoding caller as the harness of forward_prefill_logits_all / truncate_kv ----
def _plain_greedy(path, prompt, n_new):
    gm = llama_api.HipLlama(path, context_size=64)
    try:
        return gm.generate_greedy(prompt, n_new)[0]
    finally:
        gm.close()


def _draft(tokens, ngram, k):
    """Continuation of the most recent earlier occurrence of the last `ngram` tokens, at most k long."""
    n = len(tokens)
    if ngram == 0 or k == 0 or n <= ngram:
        return []
    tail = tokens[n - ngram:]
    for start in range(n - ngram - 1, -1, -1):
        if tokens[start:start + ngram] == tail:
            return tokens[start + ngram:start + ngram + k]
    return []


def _speculative_greedy(gm, prompt, max_new, ngram, k):
    """Draft from the token history, verify the draft in ONE all-logits pass, keep the longest
    prefix the model itself would have produced, roll the cache back past the rejected rest."""
    seq = list(prompt)
    logits = gm.forward_prefill(prompt, 0)
    out, rounds, drafted, accepted = [], 0, 0, 0
    nxt = int(np.argmax(logits))
    while len(out) < max_new:
        out.append(nxt); seq.append(nxt)
        if len(out) == max_new:
            break
        d = _draft(seq, ngram, min(k, max_new - len(out) - 1))
        base = gm.seq_len
        rows = gm.forward_prefill_logits_all([nxt] + d, base)      # row i = logits after token i of the batch
        rounds += bool(d); drafted += len(d)
        keep = 0
        while keep < len(d) and int(np.argmax(rows[keep])) == d[keep]:
            keep += 1
        accepted += keep
        out.extend(d[:keep]); seq.extend(d[:keep])
        gm.truncate_kv(base + 1 + keep)
        nxt = int(np.argmax(rows[keep]))
    return out[:max_new], dict(rounds=rounds, drafted=drafted, accepted=accepted)


def test_speculative_greedy_is_a_greedy_decode(tiny_llama):
    """cera/tests/spec_decode_logits.rs:212-330 in spirit: every emitted token is the target's own
    argmax over a row of forward_prefill_logits_all, so the stream equals the sequential greedy
    loop token for token on this small model; a drafter that never matches runs no verification
    batch longer than one token; the budget cap is exact."""
    path, cfg, _, _ = tiny_llama
    prompt = [5, 6, 7, 8] * 5
    plain = [int(t) for t in _plain_greedy(path, prompt, 30)]
    gm = llama_api.HipLlama(path, context_size=64)
    try:
        spec, st = _speculative_greedy(gm, prompt, 30, ngram=2, k=4)
        _say(f"spec: drafted {st['drafted']} accepted {st['accepted']} rounds {st['rounds']}")
        assert spec == plain
        assert st["rounds"] > 0 and 0 <= st["accepted"] <= st["drafted"]
        assert gm.seq_len <= len(prompt) + 30
        none, st0 = _speculative_greedy(gm, prompt, 30, ngram=999, k=4)   # fresh sequence at position 0
        assert none == plain and st0["rounds"] == 0 and st0["drafted"] == 0
        capped, _ = _speculative_greedy(gm, prompt, 7, ngram=2, k=4)
        assert capped == plain[:7]
    finally:
        gm.close()


def test_two_generations_with_fresh_states_and_no_truncate(tiny_llama):
    """A caller hands a new InferenceState to every generate(): position 0 starts a fresh
    sequence on the device too, without a truncate_kv in between."""
    path, cfg, _, _ = tiny_llama
    gm = llama_api.HipLlama(path, context_size=64)
    try:
        a = [int(t) for t in gm.generate_greedy([9, 8, 7], 12)[0]]
        assert gm.seq_len == 3 + 11
        b = [int(t) for t in gm.generate_greedy([9, 8, 7], 12)[0]]     # no truncate_kv(0) between the two
        assert a == b
        l1 = gm.forward(5, 0)                                           # single-token entry at position 0 as well
        assert gm.seq_len == 1
        l2 = gm.forward(5, 0)
        assert np.array_equal(l1, l2)
    finally:
        gm.close()
