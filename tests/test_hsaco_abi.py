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
    return names


def test_header_documents_the_name_scheme():
    for piece in ("cera_k_quantize_q8_0", "cera_k_rmsnorm_q8_0", "cera_k_gemv_<type>_ks<KS>_<store|add>",
                  "q4_0 | q4_1 | q8_0 | q4_k | q6_k", "1 | 2 | 4 | 8", "cera_k_decode_copy_<type>",
                  "cera_k_row_gemv_<type>_p<P>_<store|add>", "cera_k_row_gemv_long_<type>_p<P>_add",
                  "cera_k_norm_gate_up_<type>_p<P>", "cera_k_norm_qkv_<ta>_<tb>_p<P>_r<R>",
                  "q4_k_q4_k | q4_k_q6_k | q6_k_q4_k | q6_k_q6_k"):
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
    for struct, fields in (("cera_k_gemv_args", g._fields_), ("cera_k_quantize_q8_0_args", q._fields_),
                           ("cera_k_rmsnorm_q8_0_args", r._fields_), ("cera_k_decode_copy_args", d._fields_),
                           ("cera_k_row_gemv_args", w._fields_)):
        body = re.search(r"typedef struct \{([^}]*)\} " + struct + ";", HEADER, re.S).group(1)
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        declared = [re.search(r"(\w+)\s*$", d.strip()).group(1) for d in body.split(";") if d.strip()]
        assert declared == [f for f, _ in fields], (struct, declared)


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
