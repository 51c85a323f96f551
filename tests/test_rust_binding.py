"""The Rust `-sys` crate (rust/bdh-mi355x-sys, source only: no Rust toolchain here) against the C header: every
function include/bdh_mi355x.h declares must be declared in the crate's extern "C" block with the same name, in the same
order, with the same number of arguments and the same pointer/scalar shape per argument; constants must agree too."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _c_prototypes():
    text = open(os.path.join(ROOT, "include", "bdh_mi355x.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = []
    for ret, name, args in re.findall(r"(?:^|\n)\s*((?:const\s+)?[A-Za-z_][A-Za-z0-9_]*\s*\**)\s*(bdh_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text):
        args = " ".join(args.split())
        kinds = []
        if args not in ("void", ""):
            for a in args.split(","):
                a = a.strip()
                ty = re.match(r"(.*?)[A-Za-z_][A-Za-z0-9_]*$", a).group(1)
                kinds.append(_kind(ty.count("*"), "const" in ty, re.sub(r"const|\*|\s", "", ty)))
        out.append((name, kinds, ret.count("*")))
    return out, text


def _kind(stars, const, base):
    base = {"int": "i32", "int32_t": "i32", "int64_t": "i64", "float": "f32", "size_t": "usize", "uint64_t": "u64",
            "uint8_t": "u8", "uint16_t": "u16", "char": "c_char", "void": "c_void", "c_int": "i32"}.get(base, base)
    return (stars, const if stars else False, base)


def _rust_prototypes():
    text = open(os.path.join(ROOT, "rust", "bdh-mi355x-sys", "src", "lib.rs")).read()
    block = text[text.index('extern "C" {'):]
    out = []
    for name, args, ret in re.findall(r"pub fn (bdh_[a-z0-9_]+)\(([^)]*)\)\s*->\s*([^;]+);", block):
        kinds = []
        for a in [a for a in " ".join(args.split()).split(",") if a.strip()]:
            ty = a.split(":", 1)[1].strip()
            stars = ty.count("*")
            const = ty.startswith("*const")
            base = re.sub(r"\*const|\*mut|\s", "", ty)
            kinds.append(_kind(stars, const, base))
        out.append((name, kinds, ret.count("*")))
    return out, text


def test_extern_block_matches_the_header():
    c, _ = _c_prototypes()
    r, _ = _rust_prototypes()
    assert len(c) >= 30
    assert [n for n, _, _ in r] == [n for n, _, _ in c]
    for (name, ck, cret), (_, rk, rret) in zip(c, r):
        assert len(ck) == len(rk), f"{name}: {len(ck)} C arguments, {len(rk)} Rust arguments"
        assert ck == rk, f"{name}: argument shapes differ: {ck} vs {rk}"
        assert cret == rret, name


def test_constants_and_structs_match_the_header():
    _, ctext = _c_prototypes()
    _, rtext = _rust_prototypes()
    for name, value in re.findall(r"\b(BDH_[A-Z0-9_]+)\s*=\s*(-?\d+)", ctext):
        m = re.search(rf"pub const {name}: c_int = (-?\d+);", rtext)
        assert m and int(m.group(1)) == int(value), name
    for struct in ("bdh_model_config", "bdh_model_weights"):
        cfields = re.findall(r"([A-Za-z_0-9]+)\s*;", re.search(rf"typedef struct {struct} \{{(.*?)\}}", ctext, re.S).group(1))
        rfields = re.findall(r"pub ([a-z_0-9]+):", re.search(rf"pub struct {struct} \{{(.*?)\}}", rtext, re.S).group(1))
        assert cfields == rfields, struct


def test_python_binding_lists_every_header_symbol():
    from burn_dragon_amd import ffi

    c, _ = _c_prototypes()
    assert sorted(n for n, _, _ in c) == sorted(ffi.EXPORTS)


def test_wrappers_use_declared_symbols_and_the_reference_signature():
    """rust/bdh-mi355x-sys/src/wrappers.rs (uncompiled here): every bdh_* function it calls is declared in the
    extern block, the model is an owner with Drop, and forward_with_state has the signature of
    src/model/bdh.rs:309-313 over a ModelState of independent per-layer tensors (src/model/state.rs:5-15)."""
    _, rtext = _rust_prototypes()
    declared = set(re.findall(r"pub fn (bdh_[a-z0-9_]+)\(", rtext))
    wtext = open(os.path.join(ROOT, "rust", "bdh-mi355x-sys", "src", "wrappers.rs")).read()
    called = set(re.findall(r"\b(bdh_[a-z0-9_]+)\(", wtext))
    assert called and called <= declared, called - declared
    assert "bdh_model_forward_layers" in called and "bdh_model_destroy" in called
    assert re.search(r"impl<B: HipPointers> Drop for Model<B>", wtext)
    sig = re.search(r"pub fn forward_with_state\(&self, tokens: Tensor<B, 2, Int>, state: &mut ModelState<B>\)\s*->\s*Tensor<B, 3>",
                    wtext)
    assert sig, "forward_with_state must keep the reference's signature"
    assert re.search(r"pub struct ModelState<B: Backend> \{\s*pub layers: Vec<LayerState<B>>,\s*pub position: usize,", wtext)
