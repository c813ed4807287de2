"""The reference-side binding (integration/rust/) cannot be compiled here -- the image has no Rust
toolchain -- so its FFI block is checked against the C header text instead: the same symbols, the
same number of arguments, and for every argument and return value the same kind and width
(pointer, f64, u64, u32, int).  The trait implementations are checked for the reference's method
names (nabla-train/src/optim/core.rs:9-79, alg.rs:20-105, 181-252, 319-381)."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "nabla_optim.h")
BENCH_HEADER = os.path.join(ROOT, "include", "nabla_optim_bench.h")
FFI = os.path.join(ROOT, "integration", "rust", "ffi.rs")
MOD = os.path.join(ROOT, "integration", "rust", "mod.rs")


def _c_kind(decl: str) -> str:
    decl = decl.strip()
    if "*" in decl:
        return "ptr"
    base = re.sub(r"\b(const|unsigned)\b", "", decl).split()
    ty = base[0] if len(base) > 1 or base[0] in ("void",) else base[0]
    return {"double": "f64", "uint64_t": "u64", "uint32_t": "u32", "int": "int", "void": "void"}[ty]


def _rust_kind(ty: str) -> str:
    ty = ty.strip()
    if ty.startswith("*"):
        return "ptr"
    return {"f64": "f64", "u64": "u64", "u32": "u32", "c_int": "int", "i32": "int"}[ty]


def _header_decls():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read() + open(BENCH_HEADER).read(), flags=re.S)
    out = {}
    for ret, name, args in re.findall(r"\b(int|const char \*)\s*(nbo_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        args = args.strip()
        kinds = [] if args in ("", "void") else [_c_kind(a) for a in args.split(",")]
        out[name] = ("int" if ret == "int" else "ptr", kinds)
    return out


def _rust_decls():
    text = re.sub(r"//.*", "", open(FFI).read())
    block = text[text.index('extern "C" {'):]
    out = {}
    for name, args, ret in re.findall(r"pub fn (nbo_[a-z0-9_]+)\s*\(([^)]*)\)\s*->\s*([^;]+);", block):
        args = args.strip()
        kinds = [] if not args else [_rust_kind(a.split(":", 1)[1]) for a in args.split(",") if a.strip()]
        out[name] = (_rust_kind(ret), kinds)
    return out


def test_every_symbol_of_the_header_is_bound_with_the_same_signature():
    c, r = _header_decls(), _rust_decls()
    assert len(c) >= 50
    assert sorted(c) == sorted(r), (sorted(set(c) - set(r)), sorted(set(r) - set(c)))
    for name in c:
        assert c[name] == r[name], f"{name}: header {c[name]} vs ffi.rs {r[name]}"


def test_repr_c_structs_have_the_headers_fields_in_order():
    header = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    ffi = open(FFI).read()
    for c_name, rust_name in (("nbo_meta", "NboMeta"), ("nbo_scaler_state", "NboScalerState"),
                              ("nbo_step_info", "NboStepInfo")):
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (c_name, c_name), header, flags=re.S).group(1)
        c_fields = []
        for decl in body.split(";"):
            decl = decl.strip()
            if decl:
                ty, names = decl.split(None, 1)
                c_fields += [(n.strip(), {"int32_t": "i32", "double": "f64", "uint64_t": "u64", "uint32_t": "u32"}[ty])
                             for n in names.split(",")]
        rbody = re.search(r"#\[repr\(C\)\] pub struct %s \{(.*?)\}" % rust_name, ffi, flags=re.S).group(1)
        r_fields = [(n, t) for n, t in re.findall(r"pub (\w+): (\w+)", rbody)]
        assert c_fields == r_fields, (c_name, c_fields, r_fields)


def test_constants_agree_with_the_header():
    header, ffi = open(HEADER).read(), open(FFI).read()
    for name in ("NBO_DT_F32", "NBO_DT_BF16", "NBO_DT_F64", "NBO_DT_F16", "NBO_KIND_ADAMW", "NBO_KIND_ADAM",
                 "NBO_KIND_SGD", "NBO_OK", "NBO_ERR_LEN_MISMATCH", "NBO_ERR_COUNT_MISMATCH", "NBO_ERR_SHAPE",
                 "NBO_ERR_STATE_KEY", "NBO_ERR_STATE_INDEX", "NBO_ERR_KIND"):
        c_val = int(re.search(r"\b%s = (\d+)" % name, header).group(1))
        r_val = int(re.search(r"pub const %s: \w+ = (\d+);" % name, ffi).group(1))
        assert c_val == r_val, name
    for name in ("NBO_STEP_ZERO_GRADS", "NBO_STEP_SKIP_NONFINITE", "NBO_STEP_ZERO_ON_SKIP", "NBO_ACC_CHECK_FINITE",
                 "NBO_ACC_WRITE_GRADS"):
        c_val = int(re.search(r"#define %s (\d+)u" % name, header).group(1))
        r_val = int(re.search(r"pub const %s: u32 = (\d+);" % name, ffi).group(1))
        assert c_val == r_val, name


def test_the_shim_has_the_references_interface():
    src = open(MOD).read()
    for ty in ("MiAdamW", "MiAdam", "MiSgd"):
        assert f"impl<T: Scalar> Optimizer<T, Hip> for {ty}<T>" in src
        assert f"impl<T: Scalar> OptimState<T, Hip> for {ty}<T>" in src
    # trait Optimizer / OptimState (optim/core.rs:9-79)
    for sig in ("fn step(&mut self, params: &mut [&mut Tensor<T, Hip>], grads: &[&Tensor<T, Hip>])",
                "fn reset(&mut self)", "fn set_lr(&mut self, lr: f64)", "fn kind(&self) -> OptimKind",
                "fn state_tensors(&self) -> Vec<(String, Tensor<T, Hip>)>",
                "fn load_state_tensors(&mut self, tensors: &[(String, Tensor<T, Hip>)]) -> Result<(), String>",
                "fn meta(&self) -> OptimMeta", "fn load_meta(&mut self, meta: &OptimMeta) -> Result<(), String>"):
        assert src.count(sig) >= 3, sig
    # constructors, builders and accessors (alg.rs:20-105, 181-252, 319-381)
    for sig in ("pub fn new(lr: f64, param_shapes: &[(usize, usize)]) -> Self",
                "pub fn from_params(lr: f64, params: &[&Tensor<T, Hip>]) -> Self",
                "pub fn beta1(mut self, beta1: f64) -> Self", "pub fn weight_decay(mut self, wd: f64) -> Self",
                "pub fn momentum(mut self, momentum: f64) -> Self", "pub fn momentum_value(&self) -> f64",
                "pub fn set_state(&mut self, step_count: usize, beta1: f64, beta2: f64, eps: f64, weight_decay: f64, lr: f64)",
                "pub fn set_state(&mut self, step_count: usize, beta1: f64, beta2: f64, eps: f64, lr: f64)",
                "pub fn set_state(&mut self, lr: f64, momentum: f64, weight_decay: f64)"):
        assert sig in src, sig
    # GradScaler (optim/core.rs:334-413) and the free functions
    for sig in ("pub fn unscale_and_update<T: Scalar>(&mut self, grads: &mut [Tensor<T, Hip>]) -> bool",
                "pub fn scale_factor(&self) -> f64", "pub fn state(&self) -> GradScalerState",
                "pub fn load_state(&mut self, state: &GradScalerState)",
                "pub fn clip_grad_norm<T: Scalar>(grads: &mut [Tensor<T, Hip>], max_norm: f64) -> f64",
                "pub fn zero_grad<T: Scalar>(grads: &mut [Tensor<T, Hip>])", "pub fn adamw_step<T: Scalar>("):
        assert sig in src, sig
    # the reference's error texts that the Rust side produces itself
    for text in ('"bad tensor key: {name}"', '"{prefix} index out of range: {i}"', '"missing {prefix}{i}"',
                 '"optim kind mismatch"'):
        assert text in src, text
    # every ffi function the shim calls is declared
    declared = set(_rust_decls())
    for name in set(re.findall(r"ffi::(nbo_[a-z0-9_]+)", src)):
        assert name in declared, name


def _strip_rust(text: str) -> str:
    """Rust source with comments, string and char literals blanked (lifetimes are left alone)."""
    text = re.sub(r"//[^\n]*", "", text)
    text = re.sub(r'"(?:\\.|[^"\\])*"', '""', text)
    return re.sub(r"'(?:\\.|[^'\\])'", "' '", text)


def _call_args(text: str, open_paren: int):
    """Top-level arguments of the call whose '(' is at `open_paren`."""
    depth, args, start = 0, [], open_paren + 1
    for i in range(open_paren, len(text)):
        ch = text[i]
        if ch in "([{":
            depth += 1
        elif ch in ")]}":
            depth -= 1
            if depth == 0:
                last = text[start:i].strip()
                return args + ([last] if last else [])
        elif ch == "," and depth == 1:
            args.append(text[start:i].strip())
            start = i + 1
    raise AssertionError("unbalanced call")


def test_every_call_into_the_ffi_block_passes_the_declared_number_of_arguments():
    """What a compiler would have said first: a call site in mod.rs whose argument count differs
    from the declaration in ffi.rs, a symbol that is not declared, or delimiters that do not
    balance."""
    decls = _rust_decls()
    for path in (FFI, MOD):
        text = _strip_rust(open(path).read())
        stack = []
        for ch in text:
            if ch in "([{":
                stack.append(ch)
            elif ch in ")]}":
                assert stack and stack.pop() == {")": "(", "]": "[", "}": "{"}[ch], f"{os.path.basename(path)}: unbalanced {ch}"
        assert not stack, f"{os.path.basename(path)}: unclosed {stack[-1]}"
    text = _strip_rust(open(MOD).read())
    calls = [(m.group(1), m.end() - 1) for m in re.finditer(r"ffi::(nbo_[a-z0-9_]+)\s*\(", text)]
    assert len(calls) >= 25
    for name, at in calls:
        assert name in decls, f"mod.rs calls ffi::{name}, which ffi.rs does not declare"
        got = len(_call_args(text, at))
        assert got == len(decls[name][1]), f"ffi::{name}: {got} arguments at the call site, {len(decls[name][1])} declared"
    # every entry point a drop-in needs is actually used by the shim
    used = {name for name, _ in calls}
    for name in ("nbo_optim_step", "nbo_optim_reset", "nbo_optim_set_lr", "nbo_optim_state_read", "nbo_optim_state_write",
                 "nbo_optim_get_meta", "nbo_optim_load_meta", "nbo_scaler_unscale_and_update", "nbo_clip_grad_norm",
                 "nbo_zero_grad", "nbo_fused_step"):
        assert name in used, name
