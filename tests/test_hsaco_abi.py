"""CPU checks of the lower ABI: the built code object carries every kernel name the header
documents, and the ctypes mirrors of the argument structs have the header's natural C layout."""
import ctypes as C
import re
from pathlib import Path

import pytest

from cera_amd import _build, hsaco_api

ROOT = Path(__file__).resolve().parent.parent
HEADER = (ROOT / "include" / "cera_hip_kernels.h").read_text()


def _documented_kernels():
    names = {"cera_k_quantize_q8_0", "cera_k_rmsnorm_q8_0"}
    for t in ("q4_0", "q4_1", "q8_0", "q4_k", "q6_k"):
        for ks in (1, 2, 4, 8):
            for epi in ("store", "add"):
                names.add(f"cera_k_gemv_{t}_ks{ks}_{epi}")
    kq, b32 = ("q4_k", "q6_k"), ("q4_0", "q4_1", "q8_0")
    for t in kq + b32:
        names.add(f"cera_k_decode_copy_{t}")
        for p in ((1,) if t in kq else (1, 2)):
            names.update(f"cera_k_row_gemv_{t}_p{p}_{epi}" for epi in ("store", "add"))
            if t != "q6_k":
                names.add(f"cera_k_norm_gate_up_{t}_p{p}")
        for p in ((2, 3, 4) if t in kq else (4, 8)):
            names.add(f"cera_k_row_gemv_long_{t}_p{p}_add")
    pairs = [(a, b, (1,)) for a in kq for b in kq] + [(t, t, (1, 2)) for t in b32]
    for a, b, ps in pairs:
        names.update(f"cera_k_norm_qkv_{a}_{b}_p{p}_r{r}" for p in ps for r in (1, 2))
    # the rest of a forward pass
    names.update({"cera_k_embed_token", "cera_k_embed_rows", "cera_k_rmsnorm_rows", "cera_k_rmsnorm_rows_q8_0",
                  "cera_k_rope_kv_f32", "cera_k_rope_kv_f16", "cera_k_silu_mul", "cera_k_silu_mul_q8_0", "cera_k_add",
                  "cera_k_bias", "cera_k_scale", "cera_k_argmax_partial", "cera_k_argmax_final",
                  "cera_k_gemm_act_fp8", "cera_k_gemm_act_f16", "cera_k_gemm_q4_k", "cera_k_gemm_q4_k_swiglu",
                  "cera_k_gemm_q6_k", "cera_k_gemm_q4_0", "cera_k_gemm_q4_1", "cera_k_gemm_q8_0", "cera_k_gemm_reduce"})
    for kv in ("f32", "f16"):
        for hd in (64, 128):
            names.add(f"cera_k_kv_shift_{kv}_hd{hd}")
            names.update(f"cera_k_attn_decode_partial_{kv}_hd{hd}_g{g}_s{s}" for g in (1, 2, 4) for s in (1, 4))
            names.update(f"cera_k_attn_prefill_partial_{kv}_hd{hd}_g{g}" for g in (1, 2, 4, 8))
    for hd in (64, 128):
        for q in ("", "_q8_0"):
            names.add(f"cera_k_attn_decode_merge_hd{hd}{q}")
            names.add(f"cera_k_attn_prefill_merge_hd{hd}{q}")
    return names


def test_header_documents_the_name_scheme():
    for piece in ("cera_k_quantize_q8_0", "cera_k_rmsnorm_q8_0", "cera_k_gemv_<type>_ks<KS>_<store|add>",
                  "q4_0 | q4_1 | q8_0 | q4_k | q6_k", "1 | 2 | 4 | 8", "cera_k_decode_copy_<type>",
                  "cera_k_row_gemv_<type>_p<P>_<store|add>", "cera_k_row_gemv_long_<type>_p<P>_add",
                  "cera_k_norm_gate_up_<type>_p<P>", "cera_k_norm_qkv_<ta>_<tb>_p<P>_r<R>",
                  "q4_k_q4_k | q4_k_q6_k | q6_k_q4_k | q6_k_q6_k",
                  "cera_k_embed_token / cera_k_embed_rows", "cera_k_rmsnorm_rows / cera_k_rmsnorm_rows_q8_0",
                  "cera_k_rope_kv_<f32|f16>", "cera_k_attn_decode_partial_<f32|f16>_hd<64|128>_g<1|2|4>_s<1|4>",
                  "cera_k_attn_decode_merge_hd<64|128>[_q8_0]", "cera_k_attn_prefill_partial_<f32|f16>_hd<64|128>_g<1|2|4|8>",
                  "cera_k_attn_prefill_merge_hd<64|128>[_q8_0]", "cera_k_silu_mul[_q8_0], cera_k_add, cera_k_bias, cera_k_scale",
                  "cera_k_argmax_partial / cera_k_argmax_final", "cera_k_kv_shift_<f32|f16>_hd<64|128>",
                  "cera_k_gemm_q4_k", "cera_k_gemm_q4_k_swiglu", "cera_k_gemm_q6_k", "cera_k_gemm_q4_0 | q4_1 | q8_0",
                  "cera_k_gemm_act_fp8", "cera_k_gemm_act_f16", "cera_k_gemm_reduce"):
        assert piece in HEADER, piece


def test_code_object_exports_every_documented_kernel():
    if not _build.HSACO.exists():
        pytest.fail("cera_hip_gfx950.hsaco is not built: run __graft_entry__.build()")
    blob = _build.HSACO.read_bytes()
    assert blob[:4] == b"\x7fELF"
    missing = [n for n in sorted(_documented_kernels()) if (n.encode() + b"\x00") not in blob]
    assert not missing, missing
    # and nothing under the cera_k_ prefix that the header does not document
    found = set(m.decode() for m in re.findall(rb"cera_k_[a-z0-9_]+(?=\x00)", blob))
    found = {n for n in found if not n.endswith("_kd")}
    assert found <= _documented_kernels() | {n + ".kd" for n in _documented_kernels()}, sorted(found - _documented_kernels())


def test_argument_struct_layouts():
    # natural C layout on LP64: the header's structs, field by field
    g = hsaco_api.GemvArgs
    assert C.sizeof(g) == 88
    assert [getattr(g, f).offset for f, _ in g._fields_] == [0, 8, 16, 24, 32, 40, 48, 52, 56, 60, 64, 72, 80]
    q = hsaco_api.QuantizeArgs
    assert C.sizeof(q) == 40 and [getattr(q, f).offset for f, _ in q._fields_] == [0, 8, 16, 24, 32]
    r = hsaco_api.RmsnormQ8Args
    assert C.sizeof(r) == 48 and [getattr(r, f).offset for f, _ in r._fields_] == [0, 8, 16, 20, 24, 32, 40]
    d = hsaco_api.DecodeCopyArgs
    assert C.sizeof(d) == 32 and [getattr(d, f).offset for f, _ in d._fields_] == [0, 8, 16, 20, 24]
    w = hsaco_api.RowGemvArgs
    assert C.sizeof(w) == 104
    assert [getattr(w, f).offset for f, _ in w._fields_] == [0, 8, 16, 20, 24, 28, 32, 40, 48, 56, 64, 72, 80, 88, 96]
    pr = hsaco_api.RowGemvPairArgs
    assert C.sizeof(pr) == 216 and pr.b.offset == 104 and pr.n_blocks_a.offset == 208
    # the header declares the same fields in the same order
    more = (("cera_k_embed_token_args", hsaco_api.EmbedTokenArgs), ("cera_k_embed_rows_args", hsaco_api.EmbedRowsArgs),
            ("cera_k_rmsnorm_rows_args", hsaco_api.RmsnormRowsArgs), ("cera_k_rope_kv_args", hsaco_api.RopeKvArgs),
            ("cera_k_attn_decode_args", hsaco_api.AttnDecodeArgs), ("cera_k_attn_merge_args", hsaco_api.AttnMergeArgs),
            ("cera_k_attn_prefill_args", hsaco_api.AttnPrefillArgs), ("cera_k_silu_mul_args", hsaco_api.SiluMulArgs),
            ("cera_k_argmax_partial_args", hsaco_api.ArgmaxPartialArgs), ("cera_k_argmax_final_args", hsaco_api.ArgmaxFinalArgs),
            ("cera_k_kv_shift_args", hsaco_api.KvShiftArgs), ("cera_k_gemm_args", hsaco_api.GemmArgs),
            ("cera_k_gemm_act_fp8_args", hsaco_api.GemmActFp8Args), ("cera_k_gemm_act_f16_args", hsaco_api.GemmActF16Args))
    for struct, fields in (("cera_k_gemv_args", g._fields_), ("cera_k_quantize_q8_0_args", q._fields_),
                           ("cera_k_rmsnorm_q8_0_args", r._fields_), ("cera_k_decode_copy_args", d._fields_),
                           ("cera_k_row_gemv_args", w._fields_)) + tuple((n, c._fields_) for n, c in more):
        body = re.search(r"typedef struct \{([^}]*)\} " + struct + ";", HEADER, re.S).group(1)
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        declared = []
        for decl in (x.strip() for x in body.split(";") if x.strip()):
            decl = re.sub(r"^.*?[\s\*](?=\w+(\s*,\s*\w+)*$)", "", decl)     # drop the type: "a, b, c" remain
            declared += [v.strip() for v in decl.split(",")]
        assert declared == [f for f, _ in fields], (struct, declared)


def test_new_struct_sizes_match_the_compiled_header():
    """sizeof / offsetof of the forward-pass structs as gcc lays them out, against the ctypes mirrors."""
    import subprocess, tempfile
    pairs = [("cera_k_embed_token_args", hsaco_api.EmbedTokenArgs), ("cera_k_embed_rows_args", hsaco_api.EmbedRowsArgs),
             ("cera_k_rmsnorm_rows_args", hsaco_api.RmsnormRowsArgs), ("cera_k_rope_kv_args", hsaco_api.RopeKvArgs),
             ("cera_k_attn_decode_args", hsaco_api.AttnDecodeArgs), ("cera_k_attn_merge_args", hsaco_api.AttnMergeArgs),
             ("cera_k_attn_prefill_args", hsaco_api.AttnPrefillArgs), ("cera_k_silu_mul_args", hsaco_api.SiluMulArgs),
             ("cera_k_argmax_partial_args", hsaco_api.ArgmaxPartialArgs), ("cera_k_argmax_final_args", hsaco_api.ArgmaxFinalArgs),
             ("cera_k_kv_shift_args", hsaco_api.KvShiftArgs), ("cera_k_gemm_args", hsaco_api.GemmArgs),
             ("cera_k_gemm_act_fp8_args", hsaco_api.GemmActFp8Args), ("cera_k_gemm_act_f16_args", hsaco_api.GemmActF16Args)]
    src = '#include <stdio.h>\n#include <stddef.h>\n#include "cera_hip_kernels.h"\nint main(void){'
    for name, cls in pairs:
        src += f'printf("%zu", sizeof({name}));'
        for f, _ in cls._fields_:
            src += f'printf(" %zu", offsetof({name}, {f}));'
        src += 'printf("\\n");'
    src += f'printf("%llu\\n", (unsigned long long)CERA_K_GEMM_FP8_ACT_BYTES(65, 512));return 0;}}'
    with tempfile.TemporaryDirectory() as d:
        c = Path(d) / "m.c"
        c.write_text(src)
        subprocess.run(["gcc", "-I", str(ROOT / "include"), str(c), "-o", str(Path(d) / "m")], check=True)
        lines = subprocess.run([str(Path(d) / "m")], check=True, capture_output=True, text=True).stdout.strip().split("\n")
    for (name, cls), line in zip(pairs, lines):
        got = [int(v) for v in line.split()]
        want = [C.sizeof(cls)] + [getattr(cls, f).offset for f, _ in cls._fields_]
        assert got == want, (name, got, want)
    assert int(lines[-1]) == hsaco_api.gemm_fp8_act_bytes(65, 512)


def test_decode_copy_row_bytes_follow_the_header_macro():
    """The Python mirror of CERA_K_DECODE_COPY_ROW_BYTES against the macro itself, compiled."""
    import subprocess, tempfile
    cases = [(t, k) for t in (2, 3, 8) for k in (32, 2048, 4096, 11008)] + [(t, k) for t in (12, 14) for k in (256, 4096, 14336)]
    src = '#include <stdio.h>\n#include "cera_hip_kernels.h"\nint main(void){' + "".join(
        f'printf("%u\\n", (unsigned)CERA_K_DECODE_COPY_ROW_BYTES({t}, {k}u));' for t, k in cases) + "return 0;}"
    with tempfile.TemporaryDirectory() as d:
        c = Path(d) / "m.c"
        c.write_text(src)
        subprocess.run(["gcc", "-I", str(ROOT / "include"), str(c), "-o", str(Path(d) / "m")], check=True)
        out = subprocess.run([str(Path(d) / "m")], check=True, capture_output=True, text=True).stdout.split()
    assert [int(v) for v in out] == [hsaco_api.decode_copy_row_bytes(t, k) for t, k in cases]
