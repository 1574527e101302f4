"""The lower ABI: the standalone gfx950 code object, driven with nothing but hipModuleLoad /
hipModuleLaunchKernel (cera_amd/hsaco_api.py never touches libcera_hip.so), must reproduce the
library's results bit for bit -- they are the same kernels -- and the library itself must give the
same bits when told to launch from the code object (cera_hip_ctx_create with an hsaco_path)."""
import numpy as np
import pytest

import util
from cera_amd import _build, hip_api, hsaco_api

pytestmark = pytest.mark.gpu


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint8)


@pytest.fixture(scope="module")
def host():
    h = hsaco_api.Host()
    yield h
    h.close()


def test_quantizer_from_the_code_object(hip, orc, host):
    print("hsaco: quantize_q8_0 via hipModuleLaunchKernel", flush=True)
    for k, seed in ((32, 1), (4096, 2), (14336, 3)):
        x = util.make_x(k, seed) * np.float32(3.0)
        s, q, _ = host.quantize_q8_0(x)
        rs, rq = hip.quantize_q8_0(x)
        os_, oq = orc.quantize_q8_0(x)
        assert np.array_equal(q, rq) and np.array_equal(_bits(s), _bits(rs))
        assert np.array_equal(q, oq) and np.array_equal(_bits(s), _bits(os_))


def test_rmsnorm_q8_0_from_the_code_object(hip, host):
    x = util.make_x(4096, 5) * np.float32(2.0)
    w = (1.0 + 0.1 * util.make_x(4096, 6)).astype(np.float32)
    y, s, q = host.rmsnorm_q8_0(x, w, 1e-5)
    ry, rs, rq = hip.rmsnorm_q8_0(x, w, 1e-5)
    assert np.array_equal(_bits(y), _bits(ry)) and np.array_equal(_bits(s), _bits(rs)) and np.array_equal(q, rq)


@pytest.mark.parametrize("dtype,m,k", [(util.Q4_K, 512, 4096), (util.Q4_K, 96, 14336), (util.Q6_K, 256, 4096),
                                       (util.Q6_K, 64, 14336), (util.Q4_0, 128, 4096), (util.Q4_1, 64, 2048),
                                       (util.Q8_0, 64, 4096), (util.Q4_K, 37, 256)])
def test_gemv_from_the_code_object(hip, orc, host, dtype, m, k):
    print(f"hsaco: gemv {util.NAMES[dtype]} {m}x{k} via hipModuleLaunchKernel", flush=True)
    w, _ = util.make_weights(dtype, m, k, seed=m + k)
    x = util.make_x(k, 9)
    got = host.gemv(dtype, w, m, k, x)
    lib = hip.gemv(dtype, w, x, m, k)
    assert np.array_equal(_bits(got), _bits(lib)), float(np.abs(got - lib).max())
    ref = orc.gemv(dtype, w, x, m, k)
    assert np.abs(got - ref).max() <= 1e-3 * util.rms(ref) + 1e-12
    r = util.make_x(m, 10)
    got_add = host.gemv(dtype, w, m, k, x, resid=r)
    assert np.abs(got_add - (r + ref)).max() <= 1e-3 * util.rms(ref) + 1e-6


@pytest.mark.parametrize("dtype,m,k", [(util.Q4_K, 512, 4096), (util.Q4_K, 37, 256), (util.Q6_K, 264, 4096), (util.Q6_K, 1030, 2048),
                                       (util.Q4_0, 128, 4096), (util.Q4_0, 77, 2048), (util.Q4_1, 64, 2080), (util.Q8_0, 96, 4096),
                                       (util.Q8_0, 40, 160)])
def test_row_gemv_on_a_decode_copy_from_the_code_object(hip, host, dtype, m, k):
    """cera_k_decode_copy_* + cera_k_row_gemv_*: the bits of the library's GEMV on the native bytes."""
    print(f"hsaco: row gemv {util.NAMES[dtype]} {m}x{k} on a decode copy", flush=True)
    w, _ = util.make_weights(dtype, m, k, seed=m + k)
    x, r = util.make_x(k, 19), util.make_x(m, 20)
    lib = hip.gemv(dtype, w, x, m, k)
    assert np.array_equal(_bits(host.row_gemv(dtype, w, m, k, x)), _bits(lib))
    assert np.array_equal(_bits(host.row_gemv(dtype, w, m, k, x, resid=r)), _bits(hip.gemv_add_dev(dtype, w, x, r, m, k)))


@pytest.mark.parametrize("dtype,m,k", [(util.Q6_K, 260, 14336), (util.Q4_K, 130, 14336), (util.Q4_K, 64, 8192), (util.Q6_K, 33, 11008),
                                       (util.Q4_0, 70, 11008), (util.Q4_0, 64, 6144), (util.Q4_1, 48, 8192), (util.Q8_0, 36, 14336)])
def test_long_row_gemv_on_a_decode_copy_from_the_code_object(hip, host, dtype, m, k):
    print(f"hsaco: long row gemv {util.NAMES[dtype]} {m}x{k} on a decode copy", flush=True)
    w, _ = util.make_weights(dtype, m, k, seed=m + k)
    x, r = util.make_x(k, 21), util.make_x(m, 22)
    got = host.row_gemv(dtype, w, m, k, x, resid=r)
    assert np.array_equal(_bits(got), _bits(hip.gemv_add_dev(dtype, w, x, r, m, k)))


@pytest.mark.parametrize("dtype,m,k", [(util.Q4_K, 14336, 4096), (util.Q4_K, 96, 2048), (util.Q4_0, 224, 4096), (util.Q4_1, 64, 1024),
                                       (util.Q8_0, 160, 4096)])
def test_norm_gate_up_from_the_code_object(hip, host, dtype, m, k):
    print(f"hsaco: norm + gate|up {util.NAMES[dtype]} {m}x{k}", flush=True)
    g, _ = util.make_weights(dtype, m, k, seed=3 * m + k)
    u, _ = util.make_weights(dtype, m, k, seed=5 * m + k)
    x = util.make_x(k, 23) * np.float32(2.0)
    nw = (1.0 + 0.1 * util.make_x(k, 24)).astype(np.float32)
    q, s = host.norm_gate_up(dtype, g, u, m, k, x, nw, 1e-5)
    lq, ls = hip.ffn_gate_up_fused(g, u, m, k, x, nw, 1e-5, ggml_type=dtype)
    assert np.array_equal(q, lq) and np.array_equal(_bits(s), _bits(ls))


@pytest.mark.parametrize("ta,ma,tb,mb,k,rpw", [(util.Q4_K, 5120, util.Q6_K, 1024, 4096, 2), (util.Q4_K, 6144, util.Q4_K, 8, 4096, 2),
                                                (util.Q6_K, 100, util.Q4_K, 52, 2048, 1), (util.Q6_K, 64, util.Q6_K, 64, 1024, 1),
                                                (util.Q4_0, 640, util.Q4_0, 128, 4096, 2), (util.Q8_0, 96, util.Q8_0, 32, 2048, 1),
                                                (util.Q4_1, 72, util.Q4_1, 24, 3072, 1)])
def test_norm_qkv_from_the_code_object(hip, host, ta, ma, tb, mb, k, rpw):
    print(f"hsaco: norm + qkv {util.NAMES[ta]} {ma} | {util.NAMES[tb]} {mb} x {k} r{rpw}", flush=True)
    wa, _ = util.make_weights(ta, ma, k, seed=ma + k)
    wb, _ = util.make_weights(tb, mb, k, seed=mb + k + 1)
    x = util.make_x(k, 25) * np.float32(1.5)
    nw = (1.0 + 0.1 * util.make_x(k, 26)).astype(np.float32)
    ya, yb = host.norm_qkv(ta, wa, ma, tb, wb, mb, k, x, nw, 1e-5, rows_per_wave=rpw)
    la, lb = hip.qkv_fused(ta, wa, ma, tb, wb, mb, k, x, nw, 1e-5)
    assert np.array_equal(_bits(ya), _bits(la)) and np.array_equal(_bits(yb), _bits(lb))


def test_library_launching_from_the_code_object(hip, orc):
    """cera_hip_ctx_create(device, hsaco_path): same results as the embedded kernels, kernel level
    and through a whole model."""
    from cera_amd import synth
    mod = hip_api.Context(0, hsaco_path=str(_build.HSACO))
    try:
        for dtype, m, k in ((util.Q4_K, 512, 4096), (util.Q6_K, 128, 14336), (util.Q4_0, 96, 4096), (util.Q8_0, 64, 1024)):
            w, _ = util.make_weights(dtype, m, k, seed=3)
            x = util.make_x(k, 4)
            assert np.array_equal(_bits(mod.gemv(dtype, w, x, m, k)), _bits(hip.gemv(dtype, w, x, m, k))), (dtype, m, k)
        cfg = dict(synth.TINY)
        weights = synth.make_llama(cfg, seed=12, sigma=0.05)
        ga, gb = hip_api.Model(hip, cfg, weights), hip_api.Model(mod, cfg, weights)
        tok = 5
        for pos in range(6):
            la, lb = ga.forward(tok, pos), gb.forward(tok, pos)
            assert np.array_equal(_bits(la), _bits(lb)), pos
            tok = int(orc.argmax(la))
        ga.close(); gb.close()
    finally:
        mod.close()


def _host_model_cfg():
    from cera_amd import synth
    return dict(synth.TINY, n_layers=2, hidden=512, ffn=1024, n_heads=8, n_kv_heads=2, head_dim=128, vocab=640, max_seq_len=96)


def test_whole_decode_step_from_the_code_object(hip, orc, host):
    """A pure hipModuleLaunchKernel host (cera_amd/hsaco_api.Model: no libcera_hip.so) runs the decode
    step of a small llama -- embedding, fused norm + Q|K|V, RoPE + cache append, split-K attention and
    merge, O, fused norm + gate|up + SwiGLU, down, final norm, head, argmax -- and gets the library's
    logits bit for bit, token after token (free-running greedy), and the oracle's within its bar."""
    from cera_amd import synth
    cfg = _host_model_cfg()
    weights = synth.make_llama(cfg, seed=77, sigma=0.05, norm_jitter=0.1)
    lib = hip_api.Model(hip, cfg, weights)
    om = orc.Llama(cfg, weights)
    hm = hsaco_api.Model(host, cfg, weights, n_cu=hip.device_info()[1])
    print("hsaco: whole decode step, 12 greedy tokens", flush=True)
    tok = 11
    for pos in range(12):
        a, b, o = hm.forward(tok, pos), lib.forward(tok, pos), om.forward(tok, pos)
        assert np.array_equal(_bits(a), _bits(b)), (pos, float(np.abs(a - b).max()))
        assert np.abs(a - o).max() <= 0.1 * util.rms(o)
        assert hm.argmax() == int(orc.argmax(a))
        tok = int(orc.argmax(a))
    lib.close(); om.close()


def test_batched_prefill_from_the_code_object(hip, orc, host):
    """The same host prefills 32 tokens in one pass and then 48 more on top -- embedding rows, rmsnorm +
    Q8_0 per row, the fp8 (Q4_K) and f16 (Q6_K) GEMMs with their activation-layout kernels, RoPE + append
    for the batch, the MFMA prefill attention and its merge, SwiGLU + Q8_0, residual GEMMs -- then decodes
    on top of the cache it built: logits equal to the library's (same kernels, same launch rules) and
    close to the oracle's batched route."""
    from cera_amd import synth
    cfg = _host_model_cfg()
    weights = synth.make_llama(cfg, seed=78, sigma=0.05, norm_jitter=0.1)
    lib = hip_api.Model(hip, cfg, weights)
    om = orc.Llama(cfg, weights)
    hm = hsaco_api.Model(host, cfg, weights, n_cu=hip.device_info()[1])
    prompt = [int(t) for t in util.rng(3).integers(0, cfg["vocab"], 32)]
    print("hsaco: 32-token prefill + 4 decode steps", flush=True)
    a, b, o = hm.forward_prefill(prompt, 0), lib.forward_prefill(prompt, 0), om.forward_prefill_batched(prompt, 0)
    assert np.array_equal(_bits(a), _bits(b)), float(np.abs(a - b).max())
    assert np.abs(a - o).max() <= 0.1 * util.rms(o)
    more = [int(t) for t in util.rng(4).integers(0, cfg["vocab"], 48)]
    a, b, o = hm.forward_prefill(more, 32), lib.forward_prefill(more, 32), om.forward_prefill_batched(more, 32)
    assert np.array_equal(_bits(a), _bits(b)), float(np.abs(a - b).max())
    assert np.abs(a - o).max() <= 0.1 * util.rms(o)
    tok = int(orc.argmax(b))
    for i in range(4):
        a, b = hm.forward(tok, 80 + i), lib.forward(tok, 80 + i)
        assert np.array_equal(_bits(a), _bits(b)), (i, float(np.abs(a - b).max()))
        tok = int(orc.argmax(b))
    lib.close(); om.close()


def test_a_wrong_code_object_is_refused(tmp_path):
    bad = tmp_path / "not_a_code_object.hsaco"
    bad.write_bytes(b"\x7fELF" + bytes(200))
    with pytest.raises(hip_api.HipError):
        hip_api.Context(0, hsaco_path=str(bad))
    with pytest.raises(hip_api.HipError):
        hip_api.Context(0, hsaco_path=str(tmp_path / "missing.hsaco"))
    hip_api.Context(0).close()   # and the runtime is still usable afterwards
