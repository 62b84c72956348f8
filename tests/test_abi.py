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
