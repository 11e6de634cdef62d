"""The Rust binding source (rust/loadngo-hip-compute/src/ffi.rs) against the C header it binds.

No Rust toolchain is at hand, so the binding cannot be compiled here; this keeps its declarations from
drifting: every function of include/lng_hip.h is declared once in ffi.rs with the same number of arguments
and the same kind (pointer / 64-bit integer / size / int / float / struct by value) in every position, every
struct has the header's fields in the header's order, every constant the header's value."""
import pathlib
import re

ROOT = pathlib.Path(__file__).resolve().parents[1]
HEADER = (ROOT / "include" / "lng_hip.h").read_text()
FFI = (ROOT / "rust" / "loadngo-hip-compute" / "src" / "ffi.rs").read_text()
LIB = (ROOT / "rust" / "loadngo-hip-compute" / "src" / "lib.rs").read_text()


def strip_comments(text, line_marker):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(line_marker + r".*", " ", text)


def c_kind(decl):
    """The kind of one C parameter or result type."""
    d = decl.strip()
    if d in ("void", ""):
        return "void"
    if "*" in d or d.startswith("lng_on_done"):
        return "ptr"
    base = re.sub(r"\b(const|struct|enum)\b", "", d).split()
    t = base[0]
    return {"int": "int", "size_t": "size", "uint64_t": "u64", "float": "f32", "double": "f64",
            "lng_slice": "LngSlice"}.get(t, t)


def rust_kind(ty):
    t = ty.strip()
    if t.startswith("*") or t == "LngOnDone":
        return "ptr"
    return {"c_int": "int", "usize": "size", "u64": "u64", "f32": "f32", "f64": "f64", "()": "void"}.get(t, t)


def c_functions():
    text = strip_comments(HEADER, "//")
    out = {}
    for m in re.finditer(r"([A-Za-z_][\w \*]*?)\b(lng_hip_\w+)\s*\(([^;{]*?)\)\s*;", text):
        ret, name, params = m.group(1), m.group(2), m.group(3)
        args = [] if params.strip() in ("void", "") else [p for p in params.split(",")]
        kinds = []
        for p in args:
            p = p.strip()
            p = re.sub(r"\b\w+$", "", p) if not p.endswith("*") else p  # drop the parameter's name
            kinds.append(c_kind(p))
        out[name] = (c_kind(ret), kinds)
    return out


def rust_functions():
    text = strip_comments(FFI, "//")
    out = {}
    for m in re.finditer(r"pub fn (lng_hip_\w+)\s*\((.*?)\)\s*(?:->\s*([^;]+?))?\s*;", text, flags=re.S):
        name, params, ret = m.group(1), m.group(2), m.group(3)
        kinds = [rust_kind(p.split(":", 1)[1]) for p in params.split(",") if ":" in p]
        out[name] = (rust_kind(ret or "()"), kinds)
    return out


def test_every_function_of_the_header_is_bound_with_the_same_kinds():
    c, r = c_functions(), rust_functions()
    assert len(c) >= 39
    assert sorted(c) == sorted(r)
    for name in c:
        assert c[name] == r[name], (name, c[name], r[name])


def c_structs():
    text = strip_comments(HEADER, "//")
    out = {}
    for m in re.finditer(r"typedef struct (\w+) \{(.*?)\} \1;", text, flags=re.S):
        fields = []
        for decl in m.group(2).split(";"):
            decl = decl.strip()
            if not decl:
                continue
            ptr = "*" in decl
            names = [n.strip().lstrip("*") for n in re.sub(r"^[\w\s]+?(?=[\*\w]+\s*(,|$))", "", decl).split(",")]
            kind = "ptr" if ptr else c_kind(re.sub(r"[\w\*]+\s*(,\s*[\w\*]+\s*)*$", "", decl))
            fields += [(n, kind) for n in names]
        out[m.group(1)] = fields
    return out


def rust_structs():
    text = strip_comments(FFI, "//")
    out = {}
    for m in re.finditer(r"#\[repr\(C\)\]\s*(?:#\[derive\([^\)]*\)\]\s*)?pub struct (\w+) \{(.*?)\}", text, flags=re.S):
        fields = [(n, rust_kind(t)) for n, t in re.findall(r"pub (\w+):\s*([^,\n]+)", m.group(2))]
        out[m.group(1)] = fields
    return out


PAIRS = {"lng_slice": "LngSlice", "lng_grouped_shape": "LngGroupedShape", "lng_completed": "LngCompleted",
         "lng_decode_item": "LngDecodeItem", "lng_prepare_item": "LngPrepareItem",
         "lng_prepare_buffers": "LngPrepareBuffers", "lng_q8_matrix": "LngQ8Matrix"}


def test_every_struct_has_the_headers_fields_in_order():
    c, r = c_structs(), rust_structs()
    assert sorted(c) == sorted(PAIRS)
    for cname, rname in PAIRS.items():
        assert c[cname] == r[rname], (cname, c[cname], r[rname])


def test_constants_agree():
    def c_enum(name):
        return int(re.search(name + r"\s*=\s*(-?\d+)", HEADER).group(1))

    for name in ("LNG_OK", "LNG_ERR_NO_DEVICE", "LNG_ERR_COMPILE", "LNG_ERR_ALLOC", "LNG_ERR_DISPATCH", "LNG_ERR_GPU",
                 "LNG_F32", "LNG_BF16"):
        assert int(re.search(r"pub const " + name + r": c_int = (-?\d+);", FFI).group(1)) == c_enum(name)
    for name in ("LNG_STATIC_SCRATCH_SLOTS", "LNG_STATIC_MAX_ROW_HEADS"):
        want = int(re.search(r"#define " + name + r" (\d+)u", HEADER).group(1))
        assert int(re.search(r"pub const " + name + r": u32 = (\d+);", FFI).group(1)) == want
    assert "pub const LNG_WINDOW_FULL: u64 = u64::MAX;" in FFI and "#define LNG_WINDOW_FULL UINT64_MAX" in HEADER
    assert "pub const LNG_NO_SINKS: u64 = u64::MAX;" in FFI and "#define LNG_NO_SINKS UINT64_MAX" in HEADER


def test_the_safe_layer_uses_every_bound_function_and_keeps_the_reference_surface():
    """Every entry point is reachable from lib.rs, and the methods gpt-oss/src/gpu.rs calls on metal-compute
    (metal-compute/src/lib.rs:35-53, apple.rs) exist under the same names."""
    for name in rust_functions():
        assert "ffi::" + name in LIB, name
    for item in ("pub struct Gpu", "pub struct Buffer", "pub struct Resident", "pub struct Slice", "pub struct GroupedShape",
                 "pub struct Completed", "pub struct Batch<'g>", "pub enum Dispatch", "pub enum Error",
                 "pub fn new() -> Result<Self, Error>", "pub fn buffer(&self, len: usize) -> Result<Buffer, Error>",
                 "pub fn resident(&self, bytes: &[u8]) -> Result<Arc<Resident>, Error>",
                 "pub fn batch(&self, buffers: Vec<Buffer>, _dispatch: Dispatch) -> Result<Batch<'_>, Error>",
                 "pub fn attach(&mut self, resident: &Arc<Resident>) -> Slice", "pub fn attention_grouped(",
                 "pub fn attention_grouped_with_sinks(", "pub fn attention_grouped_tiled(",
                 "pub fn attention_grouped_tiled_with_sinks(", "pub fn copy_rows(", "pub fn rmsnorm_rows(", "pub fn add_rows(",
                 "pub fn rotate_halves(", "pub fn rotate_halves_partial(", "pub fn gemv_q8_0(", "pub fn gemm_q8_0(",
                 "pub fn gemm_q8_0_tiled(", "pub fn barrier(&mut self)",
                 "pub fn commit<P, F>(mut self, proactor: &ProactorHandle<P>, on_done: F)"):
        assert item in LIB, item
