"""The reference-side integration files under integration/ (the cera-hip-sys crate, the Model
implementation, the patch to cera's own files) are complete files, and they agree with the C
header they bind: every entry point of include/cera_hip.h is declared in the crate's extern
block with the same name, the same number of arguments and the corresponding Rust types.
No Rust toolchain exists in the build image, so this consistency check is what can be run."""
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = (ROOT / "include" / "cera_hip.h").read_text()
SYS = (ROOT / "integration" / "cera-hip-sys" / "src" / "lib.rs").read_text()
MODEL = (ROOT / "integration" / "cera" / "src" / "model" / "hip_llama.rs").read_text()
PATCH = (ROOT / "integration" / "cera-hip-backend.patch").read_text()

SCALARS = {"int": "c_int", "uint32_t": "u32", "uint64_t": "u64", "int32_t": "i32", "int8_t": "i8", "uint8_t": "u8", "uint16_t": "u16",
           "float": "f32", "char": "c_char", "cera_hip_status": "cera_hip_status", "void": "c_void"}


def _c_to_rust(ctype: str) -> str:
    words = ctype.replace("*", " * ").split()
    const = "const" in words
    stars = words.count("*")
    base = [w for w in words if w not in ("const", "*")]
    assert len(base) == 1, ctype
    r = SCALARS.get(base[0], base[0])
    for i in range(stars):
        r = ("*const " if const and i == 0 else "*mut ") + r
    return r


def _header_prototypes():
    src = re.sub(r"/\*.*?\*/", "", HEADER, flags=re.S)
    out = {}
    for proto in re.findall(r"CERA_HIP_API\s+(.*?);", src, flags=re.S):
        if "__attribute__" in proto:
            continue
        proto = " ".join(proto.split())
        m = re.match(r"(.+?)\s*\b(cera_hip_\w+)\s*\((.*)\)$", proto)
        ret, name, args = m.group(1).strip(), m.group(2), m.group(3)
        types = []
        for a in args.split(","):
            a = a.strip()
            # drop the parameter name when there is one (an identifier that is not a type word)
            m2 = re.match(r"(.*[\s\*])(\w+)$", a)
            if m2 and m2.group(2) not in SCALARS and not m2.group(2).startswith("cera_hip_") and m2.group(1).strip() not in ("const",):
                a = m2.group(1)
            types.append(_c_to_rust(a))
        out[name] = (types, None if ret == "void" else _c_to_rust(ret))
    return out


def _rust_prototypes():
    block = re.search(r'unsafe extern "C" \{(.*?)\n\}', SYS, re.S).group(1)
    out = {}
    for m in re.finditer(r"pub fn (\w+)\((.*?)\)\s*(?:->\s*([^;]+))?;", block, re.S):
        name, args, ret = m.group(1), m.group(2), m.group(3)
        types = [" ".join(a.split(":", 1)[1].split()) for a in args.split(",") if a.strip()]
        out[name] = (types, ret.strip() if ret else None)
    return out


def test_extern_block_matches_the_header():
    h, r = _header_prototypes(), _rust_prototypes()
    assert len(h) >= 60
    assert sorted(h) == sorted(r), (sorted(set(h) - set(r)), sorted(set(r) - set(h)))
    for name in h:
        assert len(h[name][0]) == len(r[name][0]), (name, h[name], r[name])
        assert h[name] == r[name], (name, h[name], r[name])


def test_struct_fields_match_the_header():
    src = re.sub(r"/\*.*?\*/", "", HEADER, flags=re.S)
    for struct in ("cera_hip_tensor", "cera_hip_layer", "cera_hip_config", "cera_hip_gemv_op", "cera_hip_decode_op"):
        body = re.search(r"typedef struct \{([^}]*)\} " + struct + ";", src).group(1)
        c_fields = []
        for decl in body.split(";"):
            decl = decl.strip()
            if decl:
                c_fields += [re.sub(r"[\s\*]", "", part.split()[-1]) for part in decl.split(",")]
        rs = re.search(r"pub struct " + struct + r" \{(.*?)\n\}", SYS, re.S).group(1)
        r_fields = re.findall(r"pub (\w+):", rs)
        assert c_fields == r_fields, (struct, c_fields, r_fields)


def test_status_codes_and_type_ids_match_the_header():
    for name, val in re.findall(r"(CERA_HIP_(?:OK|ERR_\w+|F32|F16|BF16|Q\w+))\s*=\s*(\d+)", HEADER):
        m = re.search(r"pub const " + name + r": \w+ = (\d+);", SYS)
        assert m and m.group(1) == val, name


def test_model_file_uses_only_declared_entry_points_and_overrides_trait_methods():
    declared = set(_rust_prototypes())
    used = set(re.findall(r"sys::(cera_hip_\w+)\(", MODEL))
    assert used and used <= declared, sorted(used - declared)
    for needed in ("cera_hip_ctx_create", "cera_hip_model_create", "cera_hip_forward", "cera_hip_forward_greedy",
                   "cera_hip_forward_prefill", "cera_hip_forward_prefill_logits_all", "cera_hip_truncate_kv",
                   "cera_hip_shift_kv", "cera_hip_configure_kv", "cera_hip_read_kv", "cera_hip_write_kv",
                   "cera_hip_set_seq_len", "cera_hip_memory_bytes", "cera_hip_model_destroy", "cera_hip_ctx_destroy"):
        assert needed in used, needed
    for method in ("fn forward(", "fn forward_prefill(", "fn forward_prefill_logits_all(", "fn supports_all_logits(",
                   "fn truncate_kv(", "fn config(", "fn supports_kv_shift(", "fn shift_kv(", "fn forward_greedy(",
                   "fn gpu_memory_bytes(", "fn snapshot_state(", "fn restore_state(", "fn f16_kv_supported(",
                   "fn configure_kv_compression("):
        assert method in MODEL, method


def test_files_are_complete():
    for text in (SYS, MODEL, PATCH, (ROOT / "integration" / "cera-hip-sys" / "build.rs").read_text(),
                 (ROOT / "integration" / "cera-hip-sys" / "Cargo.toml").read_text()):
        for marker in ("…", "/* ... */", "todo!(", "unimplemented!("):
            assert marker not in text.replace('unimplemented!("', "X"), marker   # quoted trait docs aside
    for text in (MODEL, SYS):
        code = re.sub(r"//[^\n]*", "", text)   # comments may hold half-open intervals
        assert code.count("{") == code.count("}") and code.count("(") == code.count(")")


def _hunks(patch: str):
    cur, old_start, old_lines = None, None, None
    for line in patch.splitlines():
        if line.startswith("--- a/"):
            cur = line[6:].strip()
        elif line.startswith("+++ ") or line.startswith("diff "):
            continue
        elif line.startswith("@@"):
            if old_lines is not None:
                yield f, old_start, old_lines
            f = cur
            old_start = int(re.match(r"@@ -(\d+)", line).group(1))
            old_lines = []
        elif old_lines is not None and (line.startswith(" ") or line.startswith("-") or line == ""):
            old_lines.append(line[1:] if line else "")
    if old_lines is not None:
        yield f, old_start, old_lines


def test_patch_touches_the_expected_files():
    files = set(re.findall(r"^\+\+\+ b/(\S+)", PATCH, re.M))
    assert {"Cargo.toml", "cera/Cargo.toml", "cera-cli/Cargo.toml", "cera/src/engine.rs", "cera/src/model/mod.rs",
            "cera/src/model/llama.rs", "cera-cli/src/main.rs"} <= files, files
    assert "BackendPreference::Hip" in PATCH and "load_model_hip" in PATCH and 'hip = ["dep:cera-hip-sys"]' in PATCH


def test_patch_applies_to_the_reference_tree():
    ref = Path("/root/reference")
    if not ref.exists():
        pytest.skip("the reference tree is not present on this machine")
    n = 0
    for f, start, old in _hunks(PATCH):
        have = (ref / f).read_text().splitlines()
        assert have[start - 1:start - 1 + len(old)] == old, (f, start)
        n += 1
    assert n >= 20
