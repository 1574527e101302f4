"""GGUF v3 reader / writer and the synthetic-model generator (CPU only).

The reader is pinned against byte buffers laid out by hand from the format
rules the reference parser implements (cera/src/gguf.rs:409-568): magic
0x46554747, version 3, KV table, tensor infos, data section aligned to
`general.alignment` (default 32), offsets relative to it.  The writer is then
pinned by reading back what it wrote (cera/src/convert/writer.rs:205-276).
"""
import ctypes
import struct
from pathlib import Path

import numpy as np
import pytest

import util
from cera_amd import _build, host_api as H, llama_api, synth


def s(x: str) -> bytes:
    b = x.encode()
    return struct.pack("<Q", len(b)) + b


def kv_u32(k, v): return s(k) + struct.pack("<II", 4, v)
def kv_f32(k, v): return s(k) + struct.pack("<If", 6, v)
def kv_str(k, v): return s(k) + struct.pack("<I", 8) + s(v)
def kv_i32(k, v): return s(k) + struct.pack("<Ii", 5, v)


def tinfo(name, dims, ggml_type, offset):
    return s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + \
        struct.pack("<IQ", ggml_type, offset)


def build(kvs, tensors, payload=b"", version=3, magic=b"GGUF", align=32):
    head = magic + struct.pack("<IQQ", version, len(tensors), len(kvs)) + b"".join(kvs) + b"".join(tensors)
    pad = (-len(head)) % align
    return head + b"\0" * pad + payload


def test_hand_built_file_parses():
    vec = np.arange(8, dtype=np.float32)
    q8 = np.arange(34 * 4, dtype=np.uint8)            # 2 rows x 64 elements of Q8_0
    payload = vec.tobytes() + q8.tobytes()
    data = build([kv_str("general.architecture", "llama"), kv_u32("llama.block_count", 7),
                  kv_f32("llama.rope.freq_base", 500000.0), kv_i32("some.int", -5),
                  s("arr") + struct.pack("<IIQ", 9, 4, 3) + struct.pack("<III", 1, 2, 3)],
                 [tinfo("v", [8], 0, 0), tinfo("w", [64, 2], 8, 32)], payload)
    g = H.Gguf(data=data)
    assert g.get_str("general.architecture") == "llama"
    assert g.get_u32("llama.block_count") == 7
    assert g.get_f32("llama.rope.freq_base") == 500000.0
    # typed getters accept exactly one value type (gguf.rs:578-600)
    assert g.get_u32("some.int") is None and g.get_f32("llama.block_count") is None
    assert g.get_u32("llama.rope.freq_base") is None and g.get_str("llama.block_count") is None
    assert g.get_u32("absent") is None
    assert g.data_offset % 32 == 0
    assert g.tensor_names() == ["v", "w"]
    tv, tw = g.tensor_info("v"), g.tensor_info("w")
    assert tv["dims"] == [8] and tv["size_bytes"] == 32 and tv["offset"] == g.data_offset
    assert tw["dims"] == [64, 2] and tw["size_bytes"] == 2 * 2 * 34 and tw["offset"] == g.data_offset + 32
    assert np.array_equal(g.tensor_bytes("v").view(np.float32), vec)
    assert np.array_equal(g.tensor_bytes("w"), q8)


def test_alignment_key_moves_the_data_section():
    payload = np.ones(4, np.float32).tobytes()
    data = build([kv_u32("general.alignment", 256)], [tinfo("v", [4], 0, 0)], payload, align=256)
    g = H.Gguf(data=data)
    assert g.data_offset % 256 == 0 and g.data_offset > 0
    assert np.array_equal(g.tensor_bytes("v").view(np.float32), np.ones(4, np.float32))


@pytest.mark.parametrize("data,needle", [
    (b"", "too small"),
    (b"GGUF" + b"\0" * 8, "too small"),
    (build([], [], magic=b"GGML"), "not a GGUF file"),
    (build([], [], version=2), "unsupported GGUF version 2"),
    (build([kv_u32("a", 1)], [])[:30], "unexpected end"),
    (build([], [tinfo("t", [4], 0, 0)], b"\0" * 8), "extends beyond file"),
    (build([], [tinfo("t", [1] * 9, 0, 0)], b"\0" * 64), "too many dimensions"),
    (build([], [tinfo("t", [48], 8, 0)], b"\0" * 64), "not divisible by block size"),
    (build([kv_u32("general.alignment", 0)], []), "invalid GGUF alignment"),
    (build([s("k") + struct.pack("<I", 99)], []), "unknown GGUF metadata value type"),
])
def test_malformed_input_is_an_error(data, needle):
    with pytest.raises(H.GgufError) as e:
        H.Gguf(data=data)
    assert needle in str(e.value)


def test_unsupported_tensor_type_is_listed_but_not_loadable():
    # Q5_0 (type 6) is parseable but unmapped: size 0 marks it (gguf.rs:517-527)
    data = build([], [tinfo("t", [32], 6, 0)], b"\0" * 64)
    g = H.Gguf(data=data)
    t = g.tensor_info("t")
    assert t["ggml_type"] == 6 and t["size_bytes"] == 0 and not t["data"]


def test_writer_reader_round_trip(tmp_path):
    rng = np.random.default_rng(5)
    a = rng.standard_normal((3, 256), dtype=np.float32)
    qa = H.quantize(H.Q4_K, a)
    qb = H.quantize(H.Q8_0, rng.standard_normal((5, 32), dtype=np.float32))   # 170 bytes: forces padding
    v = rng.standard_normal(7, dtype=np.float32)                               # 28 bytes: forces padding
    w = H.GgufWriter()
    w.add_str("general.architecture", "llama")
    w.add_u32("llama.block_count", 2)
    w.add_f32("llama.attention.layer_norm_rms_epsilon", 1e-5)
    w.add_tensor("b", [32, 5], H.Q8_0, qb)
    w.add_tensor("v", [7], H.F32, v)
    w.add_tensor("a", [256, 3], H.Q4_K, qa)
    path = tmp_path / "rt.gguf"
    w.write(str(path))
    raw = path.read_bytes()
    assert raw[:4] == b"GGUF" and struct.unpack("<I", raw[4:8])[0] == 3
    with H.Gguf(str(path)) as g:
        assert g.get_u32("llama.block_count") == 2
        assert g.get_f32("llama.attention.layer_norm_rms_epsilon") == np.float32(1e-5)
        assert np.array_equal(g.tensor_bytes("a"), qa)
        assert np.array_equal(g.tensor_bytes("b"), qb)
        assert np.array_equal(g.tensor_bytes("v").view(np.float32), v)
        offs = [g.tensor_info(n)["offset"] - g.data_offset for n in ("b", "v", "a")]
        assert offs == [0, 192, 224]            # each payload starts on the next 32-byte boundary
        # the last payload is padded too (writer.rs:264-276 pads after every tensor)
        assert len(raw) == g.data_offset + 224 + (qa.size + 31) // 32 * 32


def test_synth_is_seeded_and_thread_count_invariant(tmp_path):
    cfg = dict(synth.TINY)
    p1, p2, p3 = (str(tmp_path / f"{i}.gguf") for i in range(3))
    H.synth_llama_gguf(p1, cfg, seed=9, n_threads=1)
    H.synth_llama_gguf(p2, cfg, seed=9, n_threads=5)
    H.synth_llama_gguf(p3, cfg, seed=10, n_threads=5)
    b1, b2, b3 = (open(p, "rb").read() for p in (p1, p2, p3))
    assert b1 == b2
    assert b1 != b3 and len(b1) == len(b3)


def test_synth_metadata_shapes_and_weight_statistics(tmp_path):
    cfg = dict(synth.TINY)
    path = str(tmp_path / "m.gguf")
    H.synth_llama_gguf(path, cfg, seed=2, sigma=0.02)
    g = H.Gguf(path)
    rcfg, w = g.llama_weights()
    for k in ("n_layers", "hidden", "ffn", "n_heads", "n_kv_heads", "head_dim", "vocab", "max_seq_len"):
        assert rcfg[k] == cfg[k], k
    assert rcfg["rope_type"] == 1 and rcfg["rope_theta"] == cfg["rope_theta"]
    q_dim, kv_dim = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    expect = {"token_embd.weight": (H.Q4_K, cfg["vocab"], cfg["hidden"]),
              "output.weight": (H.Q6_K, cfg["vocab"], cfg["hidden"]),
              "blk.1.attn_q.weight": (H.Q4_K, q_dim, cfg["hidden"]),
              "blk.1.attn_k.weight": (H.Q4_K, kv_dim, cfg["hidden"]),
              "blk.1.attn_v.weight": (H.Q6_K, kv_dim, cfg["hidden"]),
              "blk.0.attn_output.weight": (H.Q4_K, cfg["hidden"], q_dim),
              "blk.0.ffn_gate.weight": (H.Q4_K, cfg["ffn"], cfg["hidden"]),
              "blk.0.ffn_down.weight": (H.Q6_K, cfg["hidden"], cfg["ffn"])}
    for name, (t, m, k) in expect.items():
        assert w[name][:3] == (t, m, k), name
        assert w[name][3].size == H.row_bytes(t, k) * m
    assert np.all(w["blk.0.attn_norm.weight"] == 1.0) and w["output_norm.weight"].size == cfg["hidden"]
    # dequantized matrices are N(0, 0.02) up to quantization noise
    t, m, k, blocks = w["blk.0.ffn_down.weight"]
    deq = util.dequant_np(t, blocks, m, k)
    assert abs(float(deq.mean())) < 5e-4
    assert abs(float(deq.std()) - 0.02) < 1e-3
    # distinct tensors draw from distinct streams
    assert not np.array_equal(w["blk.0.ffn_gate.weight"][3], w["blk.0.ffn_up.weight"][3])
    assert not np.array_equal(w["blk.0.ffn_gate.weight"][3], w["blk.1.ffn_gate.weight"][3])


def test_synth_variants(tmp_path):
    cfg = dict(synth.TINY)
    path = str(tmp_path / "q.gguf")
    H.synth_llama_gguf(path, cfg, seed=4, arch="qwen3", tied_output=True, qkv_bias=True, qk_norm=True,
                       types=dict(token_embd=H.Q8_0, attn_v=H.Q4_0))
    g = H.Gguf(path)
    rcfg, w = g.llama_weights()
    assert g.get_str("general.architecture") == "qwen3" and rcfg["rope_type"] == 0
    assert "output.weight" not in w
    assert w["token_embd.weight"][0] == H.Q8_0 and w["blk.0.attn_v.weight"][0] == H.Q4_0
    assert w["blk.1.attn_q.bias"].size == cfg["n_heads"] * cfg["head_dim"]
    assert w["blk.1.attn_k_norm.weight"].size == cfg["head_dim"]
    with pytest.raises(H.GgufError):
        H.synth_llama_gguf(path, dict(cfg, hidden=96), seed=4)          # 96 is not a whole Q4_K block


def test_host_library_exports_its_c_face():
    lib = ctypes.CDLL(str(_build.HOST_LIB))
    assert not [n for n in H.HOST_SYMBOLS if not hasattr(lib, n)]


def test_llama_library_exports_its_c_face_and_needs_a_gpu(tmp_path):
    assert _build.LLAMA_LIB.exists(), "libcera_hip_llama.so missing: run __graft_entry__.build()"
    lib = ctypes.CDLL(str(_build.LLAMA_LIB))
    assert not [n for n in llama_api.LLAMA_SYMBOLS if not hasattr(lib, n)]
    # load-time checks run before any device work: a bad file is refused with its reason
    bad = tmp_path / "bad.gguf"
    bad.write_bytes(build([kv_str("general.architecture", "mamba")], []))
    with pytest.raises(llama_api.BackendError) as e:
        llama_api.HipLlama(str(bad))
    assert "mamba" in str(e.value)
    bad.write_bytes(build([kv_str("general.architecture", "llama")], []))
    with pytest.raises(llama_api.BackendError) as e:
        llama_api.HipLlama(str(bad))
    assert "missing llama.block_count" in str(e.value)


def test_reader_and_quantizers_survive_mutations_under_sanitizers(tmp_path):
    """tests/native/gguf_fuzz.cpp built with AddressSanitizer + UndefinedBehaviorSanitizer (host
    code only): 20 000 seeded mutations of a valid file must each end in an error text or in a
    file whose metadata and tensors can be walked inside the buffer, and the quantizers must take
    NaN / infinities / extreme magnitudes without an undefined conversion."""
    import subprocess
    root = Path(__file__).resolve().parent.parent
    exe = tmp_path / "gguf_fuzz"
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined,float-cast-overflow", "-fno-sanitize-recover=all",
           "-static-libasan", "-static-libubsan", f"-I{root / 'cera_amd' / 'host'}", f"-I{root / 'include'}",
           str(root / "tests" / "native" / "gguf_fuzz.cpp"), str(root / "cera_amd" / "host" / "gguf.cpp"),
           str(root / "cera_amd" / "host" / "quantize.cpp"), "-o", str(exe), "-pthread"]
    b = subprocess.run(cmd, capture_output=True, text=True)
    assert b.returncode == 0, b.stderr[-2000:]
    r = subprocess.run([str(exe), "20000"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, (r.stdout + r.stderr)[-3000:]
    assert "20000 mutations" in r.stdout and " 0 parsed" not in r.stdout
