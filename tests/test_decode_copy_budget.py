"""The rule by which a model's decode copies are handed out (cera_hip_decode_copy_plan /
cera_hip_decode_copy_reserve_bytes): plain arithmetic behind the C ABI, checked without a GPU.

The property that matters: a decode copy is an optimisation and must never be what makes a model
fail to load or to prefill.  So whatever the plan takes, the device still holds the reserve -- one
full prefill pass's buffers, its all-positions logits and the workspace headroom -- afterwards.
The reference has no counterpart (repack_q4_k_8x8, cera/src/backend/cpu.rs:1282-1358, replaces
the native bytes instead of adding a copy), so the expected values here come from the rule's own
statement in include/cera_hip.h and from sizes computed independently below.
"""
import numpy as np

from cera_amd import hip_api, synth

MiB, GiB = 1 << 20, 1 << 30


def _reserve_by_hand(c):
    """Sum of what one prefill pass allocates, written out from the model's shapes."""
    cap = min(2048, max(min(c["max_seq_len"], 2048), 64))
    q_dim, kv_dim = c["n_heads"] * c["head_dim"], c["n_kv_heads"] * c["head_dim"]
    maxk = max(c["hidden"], c["ffn"], q_dim)
    f32_rows = 2 * c["hidden"] + 2 * q_dim + 2 * kv_dim + 2 * c["ffn"]       # hidden, normed, q, attn, k, v, gate, up
    quant = cap * maxk * (1 + 2) + 2 * cap * (maxk // 32) * 4                  # int8 + f16 quants, scales, block sums
    fp8 = (cap + 63) // 64 * 2 * (maxk // 256) * 21504                         # fragment-ordered split copy
    return cap * f32_rows * 4 + quant + fp8 + cap * 4 + cap * c["vocab"] * 4 + 512 * MiB


def test_reserve_covers_a_full_prefill_pass_of_the_8b_model():
    c = dict(synth.LLAMA3_8B, max_seq_len=8192)
    r = hip_api.decode_copy_reserve_bytes(c)
    assert r == _reserve_by_hand(c)
    # 2048 x 128256 logits alone are 1.05 GB; the pass buffers ~0.5 GB
    assert 2.0e9 < r < 2.6e9


def test_reserve_shrinks_with_a_short_context():
    c = dict(synth.LLAMA3_8B, max_seq_len=256)
    assert hip_api.decode_copy_reserve_bytes(c) == _reserve_by_hand(c)
    assert hip_api.decode_copy_reserve_bytes(c) < hip_api.decode_copy_reserve_bytes(dict(c, max_seq_len=8192))
    tiny = dict(c, max_seq_len=16)   # buffers are never sized below 64 tokens
    assert hip_api.decode_copy_reserve_bytes(tiny) == _reserve_by_hand(tiny)


def test_everything_fits_on_an_empty_device():
    copies = np.array([500 * MiB] + [150 * MiB] * 192, np.uint64)
    take, used = hip_api.decode_copy_plan(copies, 280 * GiB, 3 * GiB)
    assert take.all() and used == int(copies.sum())


def test_weights_over_half_of_memory_load_with_part_of_their_copies():
    # 160 GiB of weights on a 288 GiB device: native bytes are already resident when the plan runs,
    # so 128 GiB are free; 160 GiB of copies cannot all be built, and what is built leaves the reserve
    per = 160 * GiB // 320
    copies = np.full(320, per, np.uint64)
    free, reserve = 128 * GiB, 3 * GiB
    take, used = hip_api.decode_copy_plan(copies, free, reserve)
    assert 0 < take.sum() < 320
    assert free - used >= reserve
    assert free - used - per < reserve            # and not one copy fewer than fits
    assert take[: take.sum()].all()               # handed out in priority order


def test_no_room_means_no_copies_not_an_error():
    copies = np.array([1 * GiB, 2 * GiB], np.uint64)
    take, used = hip_api.decode_copy_plan(copies, 2 * GiB, 3 * GiB)   # less free than the reserve itself
    assert not take.any() and used == 0
    take, used = hip_api.decode_copy_plan(copies, 0, 0)
    assert not take.any() and used == 0


def test_a_copy_that_does_not_fit_is_skipped_and_smaller_ones_still_tried():
    copies = np.array([4 * GiB, 0, 1 * GiB, 3 * GiB, 1 * GiB], np.uint64)   # 0: a matrix without a streaming kernel
    take, used = hip_api.decode_copy_plan(copies, 6 * GiB, 3 * GiB)
    assert take.tolist() == [False, False, True, False, True]
    assert used == 2 * GiB


def test_exact_fit_is_taken():
    take, used = hip_api.decode_copy_plan(np.array([1 * GiB], np.uint64), 4 * GiB, 3 * GiB)
    assert take.tolist() == [True] and used == 1 * GiB
    take, used = hip_api.decode_copy_plan(np.array([1 * GiB + 1], np.uint64), 4 * GiB, 3 * GiB)
    assert take.tolist() == [False]


def test_plan_against_brute_force():
    rng = np.random.default_rng(5)
    for _ in range(200):
        n = int(rng.integers(1, 12))
        copies = rng.integers(0, 8, n).astype(np.uint64) * np.uint64(256 * MiB)
        free, reserve = int(rng.integers(0, 40)) * 256 * MiB, int(rng.integers(0, 12)) * 256 * MiB
        take, used = hip_api.decode_copy_plan(copies, free, reserve)
        left, want = free, []
        for b in copies.tolist():
            ok = b > 0 and left - b >= reserve
            want.append(ok)
            if ok:
                left -= b
        assert take.tolist() == want and used == free - left
