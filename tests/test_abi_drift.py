"""Argument-list drift at the C boundary. Four statements of every entry point's argument list
exist — the C header, the ctypes table the Python mirror calls through, the Rust rows a
maintainer adds to rivoli's backend, and (for the entry points that keep a reference
signature) the reference's own prototypes — and a reordered or added `int` in any of them would
compile, pass every symbol-name check and corrupt arguments silently. Each list is parsed from
its file and compared position by position: count, name and kind."""
import glob
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "rivoli_kvcache.h")
RUST = os.path.join(ROOT, "ffi", "hip_kvcache.rs")
REFERENCE_KERNELS = "/root/reference/crates/backend/kernels"

# Entry points whose Rust rows already exist in the reference (crates/backend/src/hip_attn.rs,
# hip.rs) and bind unchanged: ffi/hip_kvcache.rs lists them in its closing comment instead of
# restating them.
REFERENCE_ROWS = {
    "rivoli_append_kv", "rivoli_index_append", "rivoli_index_topk", "rivoli_index_score", "rivoli_hash_rows",
    "rivoli_mla_attend", "rivoli_mla_attend_scratch_floats", "rivoli_device_sync", "rivoli_act_quant_f8_prefix",
    "rivoli_gather_attn_shared_kv", "rivoli_kv_compress_deposit", "rivoli_kv_compress_prefill",
    "rivoli_kv_compress_decode", "rivoli_act_quant_f4_rotated", "rivoli_index_score_blocks",
}

C_ELEM = {"float": "f32", "unsigned char": "u8", "unsigned short": "u16", "int": "i32", "unsigned int": "u32",
          "unsigned": "u32", "void": "c_void", "long long": "i64", "unsigned long long": "u64",
          "rivoli_comp_geom": "CompGeom", "rivoli_comp_finish": "CompFinish", "CompGeom": "CompGeom",
          "CompFinish": "CompFinish", "size_t": "usize", "uint32_t": "u32", "uint16_t": "u16", "uint8_t": "u8"}


def c_kind(ctype: str) -> str:
    """'const float*' -> '*const f32', 'int' -> 'i32', ..."""
    c = " ".join(ctype.replace("__restrict__", "").replace("*", " * ").split())
    if c.endswith("*"):
        base = c[:-1].strip()
        const = base.startswith("const ")
        base = base[6:] if const else base
        base = base.replace("struct ", "")
        return ("*const " if const else "*mut ") + C_ELEM.get(base, base)
    return C_ELEM.get(c, c)   # a type this library's entry points never use stays as written


def parse_c_prototypes(text: str, pattern: str, only=None):
    """{symbol: (return kind, [(kind, name), ...])} for every prototype `pattern` finds (of the
    symbols in `only`, when given)."""
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    out = {}
    for m in re.finditer(pattern, text, re.S | re.M):
        ret, sym, args = m.group(1), m.group(2), " ".join(m.group(3).split())
        if only is not None and sym not in only:
            continue
        lst = []
        if args and args != "void":
            for a in args.split(","):
                mm = re.match(r"(.*?)(\w+)$", a.strip())
                lst.append((c_kind(mm.group(1)), mm.group(2)))
        out[sym] = (C_ELEM[ret.strip()], lst)
    return out


def header_prototypes():
    return parse_c_prototypes(open(HEADER).read(), r"^(int|size_t)\s+(rivoli_\w+)\s*\(([^;{]*)\)\s*;")


def rust_rows():
    """{symbol: [(kind, name), ...]} from the launchers! rows and the extern "C" block."""
    text = re.sub(r"//[^\n]*", "", open(RUST).read())
    out = {}
    for m in re.finditer(r"(\w+)\s*->\s*(rivoli_\w+)\s*,\s*\"[^\"]+\"\s*\(([^)]*)\)\s*;", text, re.S):
        args = []
        for a in m.group(3).split(","):
            a = " ".join(a.split())
            if not a:
                continue
            name, ty = [x.strip() for x in a.split(":", 1)]
            args.append((ty.split(" as ")[-1].strip(), name))      # `usize as i32` crosses the ABI as i32
        assert m.group(2) not in out, f"two rows for {m.group(2)}"
        out[m.group(2)] = ("i32", args)
    for m in re.finditer(r"fn\s+(rivoli_\w+)\s*\(([^)]*)\)\s*->\s*(\w+)\s*;", text, re.S):
        args = []
        for a in m.group(2).split(","):
            a = " ".join(a.split())
            if a:
                name, ty = [x.strip() for x in a.split(":", 1)]
                args.append((ty, name))
        assert m.group(1) not in out, f"two declarations of {m.group(1)}"
        out[m.group(1)] = (m.group(3), args)
    return out


def test_every_header_entry_point_has_a_rust_row_with_the_same_argument_list():
    head, rust = header_prototypes(), rust_rows()
    assert len(head) >= 39
    for sym, (ret, args) in head.items():
        if sym in REFERENCE_ROWS:
            assert sym not in rust, f"{sym}: the reference already has this row"
            continue
        assert sym in rust, f"{sym}: declared in the header, no row in ffi/hip_kvcache.rs"
        r_ret, r_args = rust[sym]
        assert r_ret == ret, f"{sym}: returns {ret} in C, {r_ret} in Rust"
        assert len(r_args) == len(args), f"{sym}: {len(args)} arguments in C, {len(r_args)} in Rust"
        for i, ((ck, cn), (rk, rn)) in enumerate(zip(args, r_args)):
            assert cn.lower() == rn.lower(), f"{sym} argument {i}: `{cn}` in C, `{rn}` in Rust"
            assert ck == rk, f"{sym} argument {i} ({cn}): {ck} in C, {rk} in Rust"
    for sym in rust:
        assert sym in head, f"{sym}: a Rust row without a prototype in the header"
    # the closing comment of the Rust file names exactly the rows that bind unchanged
    listed = set(re.findall(r"^//\s+(rivoli_\w+)\s", open(RUST).read(), re.M))
    assert listed == REFERENCE_ROWS


def test_ctypes_table_matches_the_header():
    import ctypes as C

    from rivoli_amd import hip

    # (c_ulonglong and c_size_t are one class where long is 64 bits: both read as u64 here)
    kind_of = {C.c_void_p: "ptr", C.c_int: "i32", C.c_float: "f32", C.c_longlong: "i64", C.c_ulonglong: "u64"}
    head = header_prototypes()
    table = dict(hip._SIGNATURES)
    assert not set(table) & set(hip._SIZE_SIGNATURES)
    table.update(hip._SIZE_SIGNATURES)
    for sym, (ret, args) in head.items():
        assert (sym in hip._SIZE_SIGNATURES) == (ret == "usize"), f"{sym}: returns {ret}"
        assert sym in table, f"{sym}: in the header, not in rivoli_amd/hip.py"
        got = [kind_of[t] for t in table[sym]]
        want = ["ptr" if k.startswith("*") else k.replace("usize", "u64") for k, _ in args]
        assert got == want, f"{sym}: header {want}, ctypes {got}"
    for sym in table:
        assert sym in head, f"{sym}: in rivoli_amd/hip.py, not in the header"


def test_cpp_mirror_has_a_launcher_for_every_status_returning_entry_point():
    text = open(os.path.join(ROOT, "include", "rivoli_launchers.hpp")).read()
    wrapped = set(re.findall(r"RIVOLI_LAUNCHER\(\s*\w+\s*,\s*(rivoli_\w+)", text)) | set(re.findall(r"(rivoli_\w+)\(", text))
    for sym in header_prototypes():
        assert sym in wrapped, f"{sym}: no launcher in include/rivoli_launchers.hpp"


@pytest.mark.skipif(not os.path.isdir(REFERENCE_KERNELS), reason="the reference tree is not mounted")
def test_reference_signatures_are_kept_argument_for_argument():
    """Every entry point the header shares with the reference's kernels/*.hip has the reference's
    argument list: same count, same kinds, same names in the same order."""
    head = header_prototypes()
    ref = {}
    for path in sorted(glob.glob(os.path.join(REFERENCE_KERNELS, "*.hip"))):
        ref.update(parse_c_prototypes(open(path).read(),
                                      r"extern\s+\"C\"\s+(int|size_t)\s+(rivoli_\w+)\s*\(([^{;]*)\)\s*\{", only=head))
    shared = sorted(set(head) & set(ref))
    assert set(shared) >= REFERENCE_ROWS - {"rivoli_device_sync"}, sorted(REFERENCE_ROWS - set(shared))
    for sym in shared:
        (h_ret, h_args), (r_ret, r_args) = head[sym], ref[sym]
        assert h_ret == r_ret, sym
        assert [k for k, _ in h_args] == [k for k, _ in r_args], f"{sym}: kinds differ from the reference's"
        assert [n for _, n in h_args] == [n for _, n in r_args], f"{sym}: names differ from the reference's"
