"""The Rust declarations of the C ABI (rust/dp-sumcheck-sys/src/lib.rs) against the header they transcribe
(include/dpsumcheck.h), checked as text: there is no Rust toolchain here to compile them.  Every function of the
header must be declared with the same name, the same number of arguments, the same integer widths and pointer
constness and the same return type; every enum constant and #define with the same value; dps_term with the same
fields in the same order; and nothing may be declared that the header does not have.  The adapter crate's public names
are the ones the reference's call sites use."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "dpsumcheck.h")
SYS_RS = os.path.join(ROOT, "rust", "dp-sumcheck-sys", "src", "lib.rs")
ADAPTER = os.path.join(ROOT, "rust", "dp-sumcheck", "src")

C_SCALARS = {"int32_t": "i32", "uint32_t": "u32", "uint64_t": "u64", "int64_t": "i64", "int16_t": "i16", "double": "f64",
             "char": "c_char", "void": "c_void"}


def _strip_c(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def _strip_rs(text):
    return re.sub(r"//[^\n]*", "", text)


def _c_type_to_rust(t):
    """'const dps_mle *const *' -> '*const *const dps_mle' (the innermost qualifier belongs to the pointee)"""
    toks = re.findall(r"[A-Za-z_0-9]+|\*", t)
    base = [x for x in toks if x not in ("const", "*")]
    assert len(base) == 1, t
    rust = C_SCALARS.get(base[0], base[0])
    # walk left to right: a 'const' applies to what precedes it, except a leading one, which applies to the base type
    const_here = bool(toks and toks[0] == "const")
    i = 1 if const_here else 0
    while i < len(toks):
        if toks[i] == "const":
            const_here = True
        elif toks[i] == "*":
            rust = ("*const " if const_here else "*mut ") + rust
            const_here = False
        i += 1
    return rust


def c_functions():
    text = _strip_c(open(HEADER).read())
    out = {}
    for ret, name, args in re.findall(r"^\s*((?:const\s+)?[A-Za-z_0-9]+\s*\**)\s*(dps_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.M | re.S):
        params = []
        for a in [x.strip() for x in args.split(",") if x.strip()]:
            a = " ".join(a.split())
            arr = re.match(r"^(.*?)[A-Za-z_0-9]+\s*\[\d*\]$", a)  # T name[2] is T *name
            if arr:
                params.append(_c_type_to_rust(arr.group(1) + " *"))
            else:
                params.append(_c_type_to_rust(re.match(r"^(.*?)[A-Za-z_0-9]+$", a).group(1)))
        out[name] = (params, _c_type_to_rust(ret))
    return out


def rust_functions():
    text = _strip_rs(open(SYS_RS).read())
    block = re.search(r'extern "C" \{(.*)\n\}', text, flags=re.S).group(1)
    out = {}
    for name, args, ret in re.findall(r"pub fn (dps_[a-z0-9_]+)\s*\((.*?)\)\s*->\s*([^;]+);", block, flags=re.S):
        params = [" ".join(a.split(":", 1)[1].split()) for a in [x.strip() for x in args.split(",")] if a]
        out[name] = (params, " ".join(ret.split()))
    return out


def test_every_function_of_the_header_is_declared_alike():
    c, r = c_functions(), rust_functions()
    assert len(c) >= 45
    assert sorted(c) == sorted(r), (sorted(set(c) - set(r)), sorted(set(r) - set(c)))
    for name in c:
        assert c[name] == r[name], (name, c[name], r[name])


def test_constants_match():
    text = _strip_c(open(HEADER).read())
    rs = _strip_rs(open(SYS_RS).read())
    rust_consts = {k: int(v) for k, v in re.findall(r"pub const (DPS_[A-Z0-9_]+)\s*:\s*(?:i32|usize|u32)\s*=\s*(\d+)\s*;", rs)}
    c_consts = {k: int(v) for k, v in re.findall(r"#define\s+(DPS_[A-Z0-9_]+)\s+(\d+)", text)}
    for body in re.findall(r"enum\s*[a-z_]*\s*\{(.*?)\}", text, flags=re.S):
        nxt = 0
        for item in [x.strip() for x in body.split(",") if x.strip()]:
            m = re.match(r"^(DPS_[A-Z0-9_]+)(?:\s*=\s*(\d+))?$", item)
            assert m, item
            nxt = int(m.group(2)) if m.group(2) is not None else nxt
            c_consts[m.group(1)] = nxt
            nxt += 1
    assert len(c_consts) >= 25
    assert c_consts == rust_consts, (set(c_consts.items()) ^ set(rust_consts.items()))


def test_term_layout_and_callback_match():
    text = _strip_c(open(HEADER).read())
    rs = _strip_rs(open(SYS_RS).read())
    body = re.search(r"typedef struct dps_term \{(.*?)\} dps_term;", text, flags=re.S).group(1)
    c_fields = []
    for decl in [x.strip() for x in body.split(";") if x.strip()]:
        m = re.match(r"^([a-z0-9_]+)\s+([a-z_]+)(?:\[([A-Z_0-9]+)\])?$", decl)
        c_fields.append((m.group(2), C_SCALARS[m.group(1)], m.group(3)))
    rbody = re.search(r"#\[repr\(C\)\][^{]*pub struct dps_term \{(.*?)\}", rs, flags=re.S).group(1)
    r_fields = []
    for name, ty in re.findall(r"pub ([a-z_]+)\s*:\s*([^,]+),", rbody):
        arr = re.match(r"^\[([a-z0-9]+);\s*([A-Z_0-9]+)\]$", ty.strip())
        r_fields.append((name, arr.group(1), arr.group(2)) if arr else (name, ty.strip(), None))
    assert c_fields == [(n, t, {"2": "2"}.get(a, a)) for n, t, a in r_fields] or c_fields == r_fields, (c_fields, r_fields)
    # the opaque handles are all there, and the round callback has the header's five arguments
    for handle in ("dps_ctx", "dps_mle", "dps_sc", "dps_logup"):
        assert re.search(r"#\[repr\(C\)\]\s*pub struct %s \{" % handle, rs), handle
    cb = re.search(r"typedef int32_t \(\*dps_round_fn\)\((.*?)\);", text, flags=re.S).group(1)
    c_cb = [_c_type_to_rust(re.match(r"^(.*?)[A-Za-z_0-9]+$", " ".join(a.split())).group(1)) for a in cb.split(",")]
    r_cb = re.search(r"pub type dps_round_fn = Option<\s*unsafe extern \"C\" fn\((.*?)\)\s*->\s*i32,?\s*>;", rs, flags=re.S).group(1)
    assert c_cb == [" ".join(a.split(":", 1)[1].split()) for a in r_cb.split(",") if a.strip()]


def test_adapter_offers_the_names_the_reference_calls():
    # zkml/src/layers/einsum/prove.rs:164-189, zkml/src/layers/hadamard.rs:103-129, zkml/src/layers/einsum/verify.rs:159-165
    src = "\n".join(open(os.path.join(ADAPTER, f)).read() for f in sorted(os.listdir(ADAPTER)) if f.endswith(".rs"))
    for needle in ["pub struct VirtualPolynomialsBuilder", "pub fn new(_num_threads: usize, num_vars: usize)", "pub fn new_with_mles(",
                   "pub fn lift(", "pub fn to_virtual_polys(", "pub struct IOPProverState", "pub fn prove<", "pub fn get_mle_flatten_final_evaluations(",
                   "pub fn collect_raw_challenges(", "pub struct DensePolynomial", "pub fn evals<", "pub fn optimal_sumcheck_threads(",
                   "pub struct IOPProof", "pub struct IOPProverMessage", "pub fn extract_sum(", "pub fn verify<", "pub struct VPAuxInfo",
                   "pub fn zero_pad_num_vars(", "pub fn fix_high_variables(", "pub fn fix_low_variables(", "pub fn evaluate(",
                   "WitIn(u16)", "Constant(F)", "Challenge(u16, usize, F, F)", "fn append_scalars(", "fn challenge_scalar(", "fn append_and_sample("]:
        assert needle in src, needle
    # every dps_* call the adapter makes exists in the sys crate
    declared = set(rust_functions())
    used = set(re.findall(r"sys::(dps_[a-z0-9_]+)\s*\(", src))
    assert used and used <= declared, used - declared
    # braces and parentheses balance in every file (no compiler here to say so)
    for f in sorted(os.listdir(ADAPTER)) + [SYS_RS]:
        path = f if os.path.isabs(f) else os.path.join(ADAPTER, f)
        text = re.sub(r"'(\\.|[^'\\])'", "", re.sub(r'"(\\.|[^"\\])*"', '""', _strip_rs(open(path).read())))
        for a, b in ("{}", "()", "[]"):
            assert text.count(a) == text.count(b), (path, a, text.count(a), text.count(b))
