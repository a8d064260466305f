"""The source-only Rust binding (mlx-rs_amd/rust/mi-moe-sys/src/lib.rs) against include/mi_moe.h.

No Rust toolchain exists here, so the binding cannot be compiled; this test parses both files and
compares every function (name, argument order, argument types, return type), every #[repr(C)]
struct (field order and types) and the constants.  It is the check bindgen would make by
construction (mlx-sys/src/lib.rs:1-6 includes generated bindings)."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mi_moe.h")
RUST = os.path.join(ROOT, "mlx-rs_amd", "rust", "mi-moe-sys", "src", "lib.rs")

C_TO_RUST = {
    "int": "c_int", "int32_t": "i32", "int64_t": "i64", "uint32_t": "u32", "uint16_t": "u16",
    "size_t": "usize", "float": "f32", "void": "c_void", "char": "c_char",
    "mi_moe_handle": "mi_moe_handle", "mi_moe_config": "mi_moe_config",
    "mi_moe_weights": "mi_moe_weights", "mi_moe_debug_out": "mi_moe_debug_out",
    "mi_moe_qmat": "mi_moe_qmat",
}


def strip_c_comments(s):
    return re.sub(r"/\*.*?\*/", " ", s, flags=re.S)


def c_type_to_rust(t):
    """'const uint16_t *' -> '*const u16', 'int32_t' -> 'i32'."""
    t = t.strip()
    stars = t.count("*")
    base = t.replace("*", " ").split()
    const = "const" in base
    base = [b for b in base if b != "const"]
    assert len(base) == 1, t
    r = C_TO_RUST[base[0]]
    for _ in range(stars):
        r = ("*const " if const else "*mut ") + r
    return r


def parse_header():
    src = strip_c_comments(open(HEADER).read())
    funcs = {}
    for m in re.finditer(r"(?m)^((?:const\s+)?\w+\s*\*?)\s*(mi_moe_\w+)\s*\(([^;{]*?)\)\s*;", src):
        ret, name, args = m.group(1), m.group(2), m.group(3)
        args = " ".join(args.split())
        parsed = []
        if name == "mi_moe_set_error_handler":
            parsed = ["mi_moe_error_handler", "*mut c_void", "mi_moe_data_dtor"]
        elif args != "void":
            for a in args.split(","):
                a = a.strip()
                mm = re.match(r"(.*?)(\w+)$", a)  # type, then the parameter name
                parsed.append(c_type_to_rust(mm.group(1)))
        funcs[name] = (None if ret.strip() == "void" else c_type_to_rust(ret), parsed)
    structs = {}
    for m in re.finditer(r"typedef\s+struct\s*\{(.*?)\}\s*(mi_moe_\w+)\s*;", src, flags=re.S):
        fields = []
        for decl in m.group(1).split(";"):
            decl = " ".join(decl.split())
            if not decl:
                continue
            mm = re.match(r"(.*?)(\w+(?:\s*,\s*\w+)*)$", decl)
            ty = c_type_to_rust(mm.group(1))
            for nm in mm.group(2).split(","):
                fields.append((nm.strip(), ty))
        structs[m.group(2)] = fields
    consts = {m.group(1): int(m.group(2)) for m in re.finditer(r"(MI_MOE_(?:SCORE|DTYPE)_\w+)\s*=\s*(\d+)", src)}
    consts.update({m.group(1): int(m.group(2)) for m in re.finditer(r"#define\s+(MI_MOE_N_STAGES|MI_MOE_N_KERNEL_TIMES|MI_MOE_STATIC_SCRATCH_BYTES)\s+(\d+)", src)})
    return funcs, structs, consts


def parse_rust():
    src = re.sub(r"//.*", "", open(RUST).read())
    block = re.search(r'extern "C"\s*\{(.*)\}', src, flags=re.S).group(1)
    funcs = {}
    for m in re.finditer(r"pub fn (\w+)\s*\((.*?)\)\s*(?:->\s*([^;]+?))?\s*;", block, flags=re.S):
        name, args, ret = m.group(1), " ".join(m.group(2).split()), m.group(3)
        parsed = [a.split(":", 1)[1].strip() for a in args.split(",") if a.strip()]
        funcs[name] = (ret.strip() if ret else None, parsed)
    structs = {}
    for m in re.finditer(r"#\[repr\(C\)\](?:\s*#\[derive\([^)]*\)\])?\s*pub struct (\w+)\s*\{(.*?)\}", src, flags=re.S):
        fields = []
        for f in m.group(2).split(","):
            f = " ".join(f.split())
            if f.startswith("pub "):
                nm, ty = f[4:].split(":", 1)
                fields.append((nm.strip(), ty.strip()))
        structs[m.group(1)] = fields
    consts = {m.group(1): int(m.group(2)) for m in re.finditer(r"pub const (MI_MOE_\w+): \w+ = (\d+);", src)}
    return funcs, structs, consts


def test_every_header_function_is_declared_identically():
    hf, _, _ = parse_header()
    rf, _, _ = parse_rust()
    assert len(hf) == 39, sorted(hf)
    assert sorted(hf) == sorted(rf)
    for name, (ret, args) in hf.items():
        assert rf[name][0] == ret, (name, rf[name][0], ret)
        assert rf[name][1] == args, (name, rf[name][1], args)


def test_structs_have_the_same_fields_in_the_same_order():
    _, hs, _ = parse_header()
    _, rs, _ = parse_rust()
    assert sorted(hs) == ["mi_moe_config", "mi_moe_debug_out", "mi_moe_qmat", "mi_moe_weights"]
    for name, fields in hs.items():
        assert rs[name] == fields, (name, rs[name], fields)


def test_constants_agree():
    _, _, hc = parse_header()
    _, _, rc = parse_rust()
    assert len(hc) == 9
    assert hc == rc


def test_library_exports_what_the_binding_links():
    """Every symbol of the extern block is a dynamic symbol of the built library."""
    import ctypes

    lib = ctypes.CDLL(os.path.join(ROOT, "mlx-rs_amd", "libmi_moe.so"))
    rf, _, _ = parse_rust()
    for name in rf:
        assert hasattr(lib, name), name


# ---------------------------------------------------------------- the safe layer (mi-moe)
SAFE = os.path.join(ROOT, "mlx-rs_amd", "rust", "mi-moe", "src", "lib.rs")


def _safe_source():
    return re.sub(r"//.*", "", open(SAFE).read())


def _structs_with_derives(src):
    """{struct name: (set of derived traits, body text)}"""
    out = {}
    for m in re.finditer(r"((?:#\[[^\]]*\]\s*)*)(?:pub\s+)?struct\s+(\w+)\s*(?:<[^>{]*>)?\s*\{(.*?)\n    \}", src, flags=re.S):
        derives = set()
        for d in re.finditer(r"#\[derive\(([^)]*)\)\]", m.group(1)):
            derives.update(t.strip() for t in d.group(1).split(","))
        out[m.group(2)] = (derives, m.group(3))
    return out


def test_every_module_also_has_module_parameters():
    """`trait Module<Input>: ModuleParameters + Debug` (mlx-rs/src/module/module.rs:28): a type given
    an `impl Module` must derive (or implement) ModuleParameters and Debug, or it cannot compile."""
    src = _safe_source()
    structs = _structs_with_derives(src)
    impls = re.findall(r"impl\s*(?:<[^>]*>)?\s*Module<[^>]*>\s+for\s+(\w+)", src)
    assert impls, "no impl Module found"
    for name in impls:
        derives, _ = structs[name]
        has_mp = "ModuleParameters" in derives or re.search(r"impl[^{]*\bModuleParameters\s+for\s+%s\b" % name, src)
        assert has_mp, f"{name} implements Module but not ModuleParameters"
        assert "Debug" in derives, f"{name} implements Module but not Debug"


def test_parameter_fields_follow_the_checkpoint_names():
    """The flattened keys are the field names joined by dots (mlx-macros/src/module_parameters.rs:97-101):
    gate.weight and switch_mlp.{gate_proj,up_proj,down_proj}.{weight,scales,biases}."""
    structs = _structs_with_derives(_safe_source())

    def params(name):
        return re.findall(r"#\[param\]\s*pub\s+(\w+)\s*:", structs[name][1])

    assert params("SparseMoeBlock") == ["gate", "switch_mlp"]
    assert params("SwitchGlu") == ["gate_proj", "up_proj", "down_proj"]
    assert params("QuantizedSwitchLinear") == ["weight", "scales", "biases"]
    assert params("SwitchLinear") == ["weight"]
    for name in ("SparseMoeBlock", "SwitchGlu", "QuantizedSwitchLinear", "SwitchLinear"):
        assert "ModuleParameters" in structs[name][0], name


def test_derived_quantizable_types_can_be_taken_apart():
    """derive(Quantizable) rebuilds the struct from its moved-out fields
    (mlx-macros/src/quantizable.rs:76-88): such a type needs a #[quantizable] field and no Drop."""
    src = _safe_source()
    structs = _structs_with_derives(src)
    derived = [n for n, (d, _) in structs.items() if "Quantizable" in d]
    assert sorted(derived) == ["SparseMoeBlock", "SwitchGlu"]
    for name in derived:
        assert "#[quantizable]" in structs[name][1], f"{name} has no quantizable field"
        assert not re.search(r"impl\s*(?:<[^>]*>)?\s*Drop\s+for\s+%s\b" % name, src), f"{name} implements Drop"


def test_the_router_bias_reaches_the_library():
    src = _safe_source()
    assert "router_bias: std::ptr::null()" not in src
    assert re.search(r"router_bias:\s*self\.router_bias_f32", src)
