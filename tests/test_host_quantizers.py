"""Host-side GGUF quantizers (cera/src/convert/quantize.rs) checked against the
reference's own round-trip bounds and closed forms."""
import numpy as np
import pytest

import util
from cera_amd import host_api as H


def _roundtrip_err(dtype, x):
    blocks = H.quantize(dtype, x)
    return np.abs(util.dequant_np(dtype, blocks, 1, x.size)[0] - x).max()


def test_roundtrip_bounds_on_reference_fixtures():
    # convert/quantize.rs:1100-1131: sin(0.1 i), 64 values
    x = np.sin(np.arange(64, dtype=np.float32) * np.float32(0.1)).astype(np.float32)
    assert _roundtrip_err(H.Q8_0, x) < 0.05
    assert _roundtrip_err(H.Q4_0, x) < 0.20
    # convert/quantize.rs:1172-1218: sin(0.05 i) * 2, 256 values
    x = (np.sin(np.arange(256, dtype=np.float32) * np.float32(0.05)) * 2).astype(np.float32)
    assert _roundtrip_err(H.Q4_K, x) < 0.25
    assert _roundtrip_err(H.Q5_K, x) < 0.25
    assert _roundtrip_err(H.Q6_K, x) < 0.10
    # convert/quantize.rs:1220-1250: all-positive ramp 0.02 i + 1
    x = (np.arange(256, dtype=np.float32) * np.float32(0.02) + 1).astype(np.float32)
    assert _roundtrip_err(H.Q4_K, x) < 0.35
    assert _roundtrip_err(H.Q5_K, x) < 0.35


def test_q4_0_closed_form():
    # config 1 definition: d = max|w| / 8 (f16), q = floor(x/d + 8.5) clamped to 0..15
    x = util.rng(1).standard_normal(64).astype(np.float32) * 0.02
    blocks = H.quantize(H.Q4_0, x).reshape(2, 18)
    for b in range(2):
        xb = x[32 * b:32 * b + 32]
        d = np.float32(np.abs(xb).max() / np.float32(8.0)).astype(np.float16)
        assert blocks[b, 0:2].view(np.float16)[0] == d
        df = np.float32(d)
        q = np.clip(np.floor(xb * (np.float32(1.0) / df) + np.float32(8.5)), 0, 15).astype(np.uint8)
        assert np.array_equal(blocks[b, 2:], q[:16] | (q[16:] << 4))


def test_sizes_and_errors():
    assert H.tensor_bytes(H.Q4_K, 4096 * 4096) == 4096 * 2304
    assert H.tensor_bytes(H.Q6_K, 4096 * 14336) == 48168960
    assert H.tensor_bytes(H.Q4_0, 4096 * 4096) == 9437184
    assert H.tensor_bytes(H.Q4_K, 100) == 0
    with pytest.raises(ValueError):
        H.quantize(H.Q4_K, np.zeros(100, np.float32))
    z = H.quantize(H.Q4_K, np.zeros(256, np.float32))
    assert np.all(util.dequant_np(H.Q4_K, z, 1, 256) == 0)
    z = H.quantize(H.Q6_K, np.zeros(256, np.float32))
    assert np.all(util.dequant_np(H.Q6_K, z, 1, 256) == 0)


def test_threaded_equals_serial():
    x = util.rng(2).standard_normal(256 * 4096).astype(np.float32)
    for t in (H.Q4_0, H.Q8_0, H.Q4_K, H.Q5_K, H.Q6_K):
        assert np.array_equal(H.quantize(t, x, 1), H.quantize(t, x, 5))


def test_f16_matches_numpy():
    L = H.lib()
    for b in list(range(0, 65536, 7)) + [0x7BFF, 0x7C00, 0x0001, 0x03FF, 0x0400, 0x8000]:
        v = L.cera_f16_to_f32(b)
        if (b & 0x7C00) == 0x7C00 and (b & 0x3FF):
            continue
        assert np.float32(v) == np.array([b], np.uint16).view(np.float16).astype(np.float32)[0]
        assert L.cera_f32_to_f16(v) == b
