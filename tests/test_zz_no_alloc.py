"""The allocation-free decode-attention entry (cera_hip_attn_decode_dev_noalloc): its split-K
partials live in a fixed array inside the library instead of a workspace the context allocates.
Checked through the C-ABI against cera_hip_attn_decode_dev on the same device buffers: the same
kernels with the same split, so the outputs must be bit-identical -- on two calls in a row, the
second on a smaller input (the array keeps the first call's contents), and again after a call
of the allocating entry in between.  And the property the entry exists for: on a context that has
never run attention, a call leaves the device's free memory exactly where it was, while the
allocating entry on the same context visibly takes its workspace."""
import ctypes as C

import numpy as np
import pytest

import util

pytestmark = pytest.mark.gpu


def _head_major(a, L, n_kv, hd, max_seq):
    out = np.zeros((n_kv, max_seq, hd), np.float32)
    out[:, :L, :] = a.reshape(L, n_kv, hd).transpose(1, 0, 2)
    return out


def _both(hip, n_heads, n_kv, hd, L, max_seq, seed, n_splits=0):
    q = util.make_x(n_heads * hd, seed)
    k = _head_major(util.make_x(L * n_kv * hd, seed + 1), L, n_kv, hd, max_seq)
    v = _head_major(util.make_x(L * n_kv * hd, seed + 2), L, n_kv, hd, max_seq)
    dq, dk, dv = hip.to_device(q), hip.to_device(k), hip.to_device(v)
    d_out = hip.malloc(n_heads * hd * 4)
    scale = 1.0 / np.sqrt(hd)
    res = []
    for fn in (hip.lib.cera_hip_attn_decode_dev_noalloc, hip.lib.cera_hip_attn_decode_dev):
        hip.upload(d_out, np.full(n_heads * hd, np.nan, np.float32))
        print(f"no-alloc attention: {fn.__name__} heads {n_heads}/{n_kv} hd {hd} L {L} splits {n_splits}", flush=True)
        hip.check(fn(hip.h, dq, dk, dv, n_heads, n_kv, hd, L, max_seq, scale, n_splits, d_out))
        res.append(hip.download(d_out, n_heads * hd, np.float32))
    for d in (dq, dk, dv, d_out):
        hip.free(d)
    return res[0], res[1], (q, k, v)


def test_no_alloc_attention_matches_the_allocating_entry(hip, orc):
    a1, b1, (q, k, v) = _both(hip, 32, 8, 128, 4096, 4096, seed=1)              # many parts
    assert np.array_equal(a1.view(np.uint32), b1.view(np.uint32))
    ref = orc.decode_attention(q, k.transpose(1, 0, 2).reshape(-1), v.transpose(1, 0, 2).reshape(-1), 32, 8, 128,
                               1.0 / np.sqrt(128), 4096)
    assert np.abs(a1 - ref).max() <= 2e-3 * util.rms(ref)
    a2, b2, _ = _both(hip, 8, 2, 64, 37, 64, seed=9)                             # smaller, right after
    assert not np.isnan(a2).any()
    assert np.array_equal(a2.view(np.uint32), b2.view(np.uint32))
    a3, b3, _ = _both(hip, 32, 8, 128, 700, 1024, seed=5, n_splits=16)           # explicit split
    assert np.array_equal(a3.view(np.uint32), b3.view(np.uint32))


def _free_device_bytes():
    rt = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(), C.c_size_t()
    assert rt.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def test_no_alloc_attention_allocates_nothing(hip):
    from cera_amd import hip_api
    fresh = hip_api.Context(0)     # no attention workspace, no scratch slot yet
    try:
        n_heads, n_kv, hd, L = 32, 8, 128, 8192         # 128 parts x 32 heads x 128 x 4 B = 2 MiB of partials
        dq = fresh.to_device(util.make_x(n_heads * hd, 3))
        dk = fresh.to_device(np.zeros((n_kv, L, hd), np.float32))
        d_out = fresh.malloc(n_heads * hd * 4)
        fresh.sync()
        f0 = _free_device_bytes()
        print(f"no-alloc attention on a fresh context: free {f0} bytes before", flush=True)
        fresh.check(fresh.lib.cera_hip_attn_decode_dev_noalloc(fresh.h, dq, dk, dk, n_heads, n_kv, hd, L, L, 0.1, 128, d_out))
        fresh.sync()
        f1 = _free_device_bytes()
        assert f1 == f0, f"the allocation-free entry changed free device memory by {f0 - f1} bytes"
        # the probe is not blind: the allocating entry's first call on this context takes its workspace
        fresh.check(fresh.lib.cera_hip_attn_decode_dev(fresh.h, dq, dk, dk, n_heads, n_kv, hd, L, L, 0.1, 128, d_out))
        fresh.sync()
        f2 = _free_device_bytes()
        print(f"no-alloc attention: free after the allocating entry {f2} ({f1 - f2} bytes taken)", flush=True)
        assert f1 - f2 >= n_heads * 128 * hd * 4
        # and a second allocation-free call, with the context's workspace now present, still takes nothing
        fresh.check(fresh.lib.cera_hip_attn_decode_dev_noalloc(fresh.h, dq, dk, dk, n_heads, n_kv, hd, L, L, 0.1, 128, d_out))
        fresh.sync()
        assert _free_device_bytes() == f2
        for d in (dq, dk, d_out):
            fresh.free(d)
    finally:
        fresh.close()


def test_no_alloc_attention_refuses_what_does_not_fit(hip):
    # 32768 keys in 64-key chunks, one part each = 512 parts: 32 heads x 512 x 128 x 4 bytes = 8 MiB of
    # partials, beyond the fixed 4 MiB array
    L, n_kv, hd = 32768, 8, 128
    dq, dk = hip.to_device(np.zeros(32 * hd, np.float32)), hip.to_device(np.zeros((n_kv, L, hd), np.float32))
    d_out = hip.malloc(32 * hd * 4)
    st = hip.lib.cera_hip_attn_decode_dev_noalloc(hip.h, dq, dk, dk, 32, n_kv, hd, L, L, 0.1, 1024, d_out)
    assert st == 4   # CERA_HIP_ERR_SHAPE
    assert b"fixed workspace" in hip.lib.cera_hip_last_error(hip.h)
    for d in (dq, dk, d_out):
        hip.free(d)
