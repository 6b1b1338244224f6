"""The Rust binding (`custos_amd/rust/src/devices/hip/api.rs`) cannot be compiled here (no rustc),
so its extern block is checked as text against the C header: every entry point declared once,
with the same number of parameters and the same integer widths per parameter."""
import re
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
HEADER = (ROOT / "include" / "custos_hip.h").read_text()
API_RS = (ROOT / "custos_amd" / "rust" / "src" / "devices" / "hip" / "api.rs").read_text()


def split_params(text):
    text = " ".join(text.split())
    return [] if text in ("", "void") else [p.strip() for p in text.split(",")]


def c_prototypes():
    body = re.sub(r"/\*.*?\*/", "", HEADER, flags=re.S)
    out = {}
    for ret, name, params in re.findall(r"^([A-Za-z_][\w \*]*?)\s*\b(custos_hip_\w+)\s*\(([^;{]*?)\)\s*;", body, flags=re.M):
        out[name] = (" ".join(ret.split()), split_params(params))
    return out


def rust_prototypes():
    out = {}
    for name, params, ret in re.findall(r"pub fn (custos_hip_\w+)\s*\(([^)]*)\)\s*->\s*([^;]+);", API_RS):
        out[name] = (ret.strip(), split_params(params))
    return out


def c_kind(param):
    """What a C parameter is at the ABI: pointer, or a scalar of a given width."""
    if "*" in param:
        return "ptr"
    for c_type, kind in (("uint64_t", "u64"), ("int32_t", "i32"), ("uint32_t", "u32"), ("size_t", "usize"), ("double", "f64")):
        if re.search(rf"\b{c_type}\b", param):
            return kind
    raise AssertionError(f"unclassified C parameter: {param}")


def rust_kind(param):
    ty = param.split(":", 1)[1].strip()
    return "ptr" if ty.startswith("*") else ty


def test_every_entry_point_is_bound_once_with_the_same_shape():
    c, rust = c_prototypes(), rust_prototypes()
    assert len(c) > 50
    assert sorted(c) == sorted(rust), (sorted(set(c) - set(rust)), sorted(set(rust) - set(c)))
    assert len(re.findall(r"pub fn custos_hip_", API_RS)) == len(rust), "an entry point is declared twice"
    for name, (ret, params) in c.items():
        rust_ret, rust_params = rust[name]
        assert [c_kind(p) for p in params] == [rust_kind(p) for p in rust_params], name
        want_ret = {"int32_t": "i32", "uint64_t": "u64", "const char *": "*const c_char"}[ret]
        assert rust_ret == want_ret, name


def test_constants_match_the_header():
    for rust_name, c_name in (("KIND_APPLY", "CUSTOS_HIP_KIND_APPLY"), ("KIND_UNARY_GRAD", "CUSTOS_HIP_KIND_UNARY_GRAD"),
                              ("GRAPH_EDGES_LEVEL_JOINS", "CUSTOS_HIP_GRAPH_EDGES_LEVEL_JOINS"),
                              ("GRAPH_EDGES_PER_NODE", "CUSTOS_HIP_GRAPH_EDGES_PER_NODE"),
                              ("GRAPH_EDGES_CHAIN", "CUSTOS_HIP_GRAPH_EDGES_CHAIN")):
        c_value = re.search(rf"\b{c_name}\s*=\s*(\d+)", HEADER)
        rust_value = re.search(rf"pub const {rust_name}: i32 = (\d+);", API_RS)
        assert c_value and rust_value, (rust_name, c_name)
        assert c_value.group(1) == rust_value.group(1), rust_name


def test_element_type_numbers_match_the_header():
    mod_rs = (ROOT / "custos_amd" / "rust" / "src" / "devices" / "hip" / "mod.rs").read_text()
    names = {"f32": "F32", "f64": "F64", "i32": "I32", "i64": "I64", "u8": "U8", "i8": "I8", "i16": "I16", "u16": "U16",
             "u32": "U32", "u64": "U64", "half::f16": "F16_PERNODE", "half::bf16": "BF16_PERNODE"}
    for rust_type, c_name in names.items():
        c_value = re.search(rf"\bCUSTOS_HIP_{c_name}\s*=\s*(\d+)", HEADER).group(1)
        assert re.search(rf"{re.escape(rust_type)} => {c_value}\b", mod_rs), rust_type
        assert re.search(rf"TypeId::of::<{re.escape(rust_type)}>\(\)(, | \{{\s*return Some\(){c_value}\b", mod_rs), rust_type
