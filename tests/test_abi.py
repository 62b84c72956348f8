"""The C-ABI libraries load on a machine without a GPU and export every symbol the headers
declare (no compute is attempted here)."""
import ctypes as C
import os
import re

from rivoli_amd import build, hip, pagepool

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rivoli_\w+)\s*\(", text)))


def test_kvcache_header_symbols_are_exported():
    names = declared("rivoli_kvcache.h")
    assert len(names) >= 14
    lib = C.CDLL(build.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(hip.exported_symbols()) == names


def test_pagepool_header_symbols_are_exported():
    names = declared("rivoli_pagepool.h")
    names = [n for n in names if n != "rivoli_pagepool"]
    lib = C.CDLL(build.HOST_LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(pagepool.EXPORTED) == names


def test_page_bytes_is_a_pure_host_function():
    assert hip.kv_page_bytes(64, 576) == 37120
    assert hip.kv_page_bytes(0, 576) == 0


def test_status_mapping_matches_the_reference_wording():
    """crates/backend/src/hip.rs:328-336."""
    hip.ensure_hip_status(0, "x")
    for code, text in ((1002, "append_kv: argument guard rejected (1002)"),
                       (-98, "append_kv: HIP error 98")):
        try:
            hip.ensure_hip_status(code, "append_kv")
        except hip.LaunchError as e:
            assert str(e) == text and e.code == code
        else:
            raise AssertionError("no error raised")


def test_headers_compile_as_c_and_cpp(tmp_path):
    """The boundary is a C ABI: both headers are valid C11 and C++17 on their own."""
    import os
    import subprocess

    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    src = '#include "rivoli_kvcache.h"\n#include "rivoli_pagepool.h"\nint main(void) { return 0; }\n'
    for compiler, std, ext in (("gcc", "-std=c11", "c"), ("g++", "-std=c++17", "cpp")):
        f = tmp_path / f"abi.{ext}"
        f.write_text(src)
        res = subprocess.run([compiler, std, "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only", "-I", inc,
                              str(f)], capture_output=True, text=True)
        assert res.returncode == 0, res.stderr


def test_pure_host_functions_need_no_gpu():
    """Shape and sizing functions are host arithmetic (crates/engine/src/v4/select.rs Sel::shape;
    the scratch sizing convention of crates/backend/kernels/attn.hip:100-103)."""
    assert hip.sel_shape(8, 4, 512, 12, 0) == (12, 8 + 3)
    assert hip.sel_shape(128, 128, 512, 1, 300) == (1, 128 + 2)
    for args, code in (((8, 0, 512, 3, 5), 1005), ((0, 0, 512, 1, 5), 1001), ((8, 4, 2, 1, 12), 1006)):
        try:
            hip.sel_shape(*args)
            raise AssertionError(args)
        except hip.LaunchError as e:
            assert e.code == code
    assert hip.gather_attn_scratch_floats(8192, 64, 512, 640) == 0          # enough queries: no split
    assert hip.gather_attn_scratch_floats(1, 64, 512, 640) == 10 * 64 * 514   # ten shares of two tiles
    assert hip.gather_attn_scratch_floats(1, 64, 128, 640) == 0             # other widths: the plain kernel
    assert hip.compress_dst(4, 128, 1, 47) == (139, 1) and hip.compress_dst(4, 128, 1, 48) is None
