"""The Rust side of the boundary (crates/nerva-hip) cannot be compiled in this image (no cargo / rustc),
so it is checked as text against the C header the library is built from: every #[repr(C)] struct of
src/ffi.rs must have the header's fields in the header's order with types of the same size - sizes and
offsets are recomputed here under the C layout rules and compared with what ctypes computes from the
header - every entry point must be declared with the same arguments, have a stub, and the safe wrappers
may only name fields and functions that exist."""
import ctypes as C
import os
import re
import subprocess
import sys

from nerva_amd import abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CRATE = os.path.join(ROOT, "crates", "nerva-hip")

RUST_SIZES = {"i32": 4, "u32": 4, "u64": 8, "i64": 8, "u16": 2, "u8": 1, "f32": 4, "f64": 8, "c_char": 1, "c_int": 4}


def rust_structs(text):
    out = {}
    for m in re.finditer(r"#\[repr\(C\)\]\n(?:#\[derive\([^\n]*\)\]\n)?pub struct (\w+) \{(.*?)\n\}", text, flags=re.S):
        fields = re.findall(r"pub (?:r#)?(\w+): ([^,\n]+),", m.group(2))
        out[m.group(1)] = fields
    return out


def type_layout(t, structs):
    """(size, alignment) of a Rust field type under repr(C)."""
    t = t.strip()
    arr = re.match(r"\[(.+); (\d+)\]$", t)
    if arr:
        size, align = type_layout(arr.group(1), structs)
        return size * int(arr.group(2)), align
    if t.startswith("*"):
        return 8, 8
    if t in RUST_SIZES:
        return RUST_SIZES[t], RUST_SIZES[t]
    return struct_layout(t, structs)[0:2]


def struct_layout(name, structs):
    offset, align, offsets = 0, 1, []
    for field, t in structs[name]:
        size, a = type_layout(t, structs)
        offset = (offset + a - 1) // a * a
        offsets.append((field, offset, size))
        offset += size
        align = max(align, a)
    return (offset + align - 1) // align * align, align, offsets


def test_generated_files_are_current():
    rc = subprocess.run([sys.executable, os.path.join(CRATE, "generate_ffi.py"), "--check"]).returncode
    assert rc == 0, "crates/nerva-hip/src/ffi.rs or native_stubs.rs is older than include/nerva_hip_api.h: regenerate"


def test_every_repr_c_struct_has_the_headers_layout():
    structs = rust_structs(open(os.path.join(CRATE, "src", "ffi.rs")).read())
    checked = 0
    for name, ctype in abi.STRUCTS.items():
        if not getattr(ctype, "_fields_", None):
            assert name in structs and structs[name] == [] or name == "NervaHipHfDecodeSequenceSession"
            continue
        assert name in structs, "no Rust mirror of %s" % name
        size, _, offsets = struct_layout(name, structs)
        assert [f for f, _, _ in offsets] == [f for f, _ in ctype._fields_], name
        assert size == C.sizeof(ctype), (name, size, C.sizeof(ctype))
        for field, offset, fsize in offsets:
            desc = getattr(ctype, field)
            assert (offset, fsize) == (desc.offset, desc.size), (name, field, offset, fsize, desc.offset, desc.size)
        checked += 1
    assert checked >= 30
    # the sizes the reference's header gives its structs (nerva_cuda_api.h:29-37, 255-332, 436-513, 606-638)
    assert struct_layout("NervaHipSyntheticTokenSlot", structs)[0] == 40
    assert struct_layout("NervaHipHfDecodeChainLayer", structs)[0] == 440
    assert struct_layout("NervaHipHfDecodeSequenceResult", structs)[0] == 528
    assert struct_layout("NervaHipHfDecodeSequenceSessionCreateRequest", structs)[0] == 176


def test_every_entry_point_is_declared_and_stubbed():
    ffi = open(os.path.join(CRATE, "src", "ffi.rs")).read()
    stubs = open(os.path.join(CRATE, "src", "native_stubs.rs")).read()
    block = ffi[ffi.index('unsafe extern "C" {'):]
    for name, (ret, args) in abi.FUNCTIONS.items():
        m = re.search(r"pub fn %s\((.*?)\) -> (\w+);" % name, block)
        assert m, "no extern declaration of %s" % name
        n_args = 0 if args == "void" else len(args.split(","))
        assert (len(m.group(1).split(",")) if m.group(1) else 0) == n_args, name
        assert m.group(2) == {"int": "c_int", "uint64_t": "u64"}[ret], name
        assert re.search(r'#\[unsafe\(no_mangle\)\]\npub extern "C" fn %s\(' % name, stubs), "no stub for %s" % name


def test_safe_wrappers_name_only_what_exists():
    session = open(os.path.join(CRATE, "src", "session.rs")).read()
    structs = rust_structs(open(os.path.join(CRATE, "src", "ffi.rs")).read())
    for fn in set(re.findall(r"\b(nerva_hip_\w+)\(", session)):
        assert fn in abi.FUNCTIONS, fn
    # every `request.field = ...` / `layer.field = ...` / `out.field` names a field of the struct the variable has
    for decl in re.finditer(r"let mut (\w+): (NervaHip\w+) = unsafe \{ std::mem::zeroed\(\) \};(.*?)(?=\n    }\n|\n}\n)", session, flags=re.S):
        var, struct, body = decl.group(1), decl.group(2), decl.group(3)
        names = {f for f, _ in structs[struct]}
        for field in re.findall(r"\b%s\.(\w+)\b" % var, body):
            assert field in names, "%s has no field %s" % (struct, field)
    rows = open(os.path.join(CRATE, "kernel_contract_rows.patch")).read()
    contracts = open(os.path.join(CRATE, "src", "contracts.rs")).read()
    for name in re.findall(r'name: "(hip_\w+)"', contracts):
        assert '+            name: "%s",' % name in rows


def test_build_script_lists_the_sources_that_exist():
    """build.rs compiles nerva_amd/csrc/<name>.hip for every name in SOURCES: the list is the library's."""
    import re
    text = open(os.path.join(ROOT, "crates", "nerva-hip", "build.rs")).read()
    block = re.search(r"const SOURCES: &\[&str\] = &\[(.*?)\];", text, re.S).group(1)
    names = re.findall(r'"([a-z0-9_]+)"', block)
    csrc = os.path.join(ROOT, "nerva_amd", "csrc")
    assert sorted(names) == sorted(f[:-4] for f in os.listdir(csrc) if f.endswith(".hip"))


def test_safe_wrapper_checks_every_tensor_before_the_pointer_cast():
    """The config's validate() must compare every layer tensor with the size the dimensions imply (native code reads
    that many elements from the pointer it is handed) and convert sizes with checked conversions; the crate's build
    script must refuse register spills in the kernels that issue loads by hand, like nerva_amd/build.py."""
    session = open(os.path.join(CRATE, "src", "session.rs")).read()
    validate = session[session.index("pub fn validate("):session.index("pub fn create(")]
    for tensor in ("w_q", "w_k", "w_v", "w_o", "w_gate", "w_up", "w_down", "rms_attn_weight", "rms_mlp_weight",
                   "q_norm_weight", "k_norm_weight", "q_bias", "k_bias", "v_bias", "o_bias", "embeddings", "lm_head",
                   "final_norm_weight"):
        assert re.search(r"\b%s\b" % tensor, validate), "validate() does not look at %s" % tensor
    assert "checked_mul" in validate and "u32::try_from" in validate
    assert not re.search(r"\b(len\(\)|steps|self\.\w+) as u32", session), "unchecked size conversion"
    from nerva_amd import build
    script = open(os.path.join(CRATE, "build.rs")).read()
    for kernel in build.HAND_ISSUED_LOADS:
        assert '"%s"' % kernel in script
    assert "kernel-resource-usage" in script and "ScratchSize" in script and 'SUPPORTED_ARCH: &str = "gfx950"' in script
