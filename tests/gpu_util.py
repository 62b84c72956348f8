"""Device-buffer plumbing for the GPU parity tests: torch only allocates and copies."""
import ctypes as C
import os

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_LIB = os.path.join(ROOT, "oracle", "_ref", "librivoli_ref_kernels.so")


def torch_cuda():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch


def dev(a: np.ndarray):
    """Upload any numpy array as raw bytes (a uint8 device tensor)."""
    torch = torch_cuda()
    b = np.ascontiguousarray(a).view(np.uint8).reshape(-1)
    return torch.from_numpy(b.copy()).cuda()


def dzeros(nbytes: int, fill: int = 0):
    torch = torch_cuda()
    return torch.full((int(nbytes),), fill, dtype=torch.uint8, device="cuda")


def back(t, dtype=np.uint8) -> np.ndarray:
    """Synchronise and download as `dtype`."""
    return t.cpu().numpy().view(dtype)


_REF = None


def need_ref(*symbols):
    """The reference's own launchers (ref_kernels), or a SKIP when that build is not there or
    lacks one of `symbols`: a test whose only claim is "the reference's kernel agrees" must not
    read as passed on a box that never ran it."""
    ref = ref_kernels()
    if ref is None:
        pytest.skip("oracle/_ref not built: the reference's own kernels were not run")
    for name in symbols:
        if not hasattr(ref, name):
            pytest.skip(f"oracle/_ref lacks {name}: the reference's own kernel was not run")
    return ref


def ref_kernels():
    """The reference's own launchers compiled for gfx950 (oracle/Makefile `ref`), or None.
    They run on the null stream like every launch in these tests."""
    global _REF
    if _REF is None and os.path.exists(REF_LIB):
        h = C.CDLL(REF_LIB)
        vp, i = C.c_void_p, C.c_int
        h.rivoli_append_kv.restype, h.rivoli_append_kv.argtypes = i, [vp] * 5 + [i] * 4
        h.rivoli_index_append.restype, h.rivoli_index_append.argtypes = i, [vp, vp, i, i]
        h.rivoli_index_topk.restype, h.rivoli_index_topk.argtypes = i, [vp, i, i, vp]
        if hasattr(h, "rivoli_mla_attend"):
            h.rivoli_mla_attend.restype = i
            h.rivoli_mla_attend.argtypes = [vp] * 6 + [i] * 5 + [C.c_float, vp, vp]
            h.rivoli_mla_attend_scratch_floats.restype = C.c_size_t
            h.rivoli_mla_attend_scratch_floats.argtypes = [i, i]
        if hasattr(h, "rivoli_gather_attn_shared_kv"):
            h.rivoli_gather_attn_shared_kv.restype = i
            h.rivoli_gather_attn_shared_kv.argtypes = [vp] * 4 + [i] * 4 + [C.c_float, vp, vp]
        if hasattr(h, "rivoli_act_quant_f8_prefix"):
            h.rivoli_act_quant_f8_prefix.restype = i
            h.rivoli_act_quant_f8_prefix.argtypes = [vp, vp] + [i] * 4 + [vp]
        if hasattr(h, "rivoli_kv_compress_prefill"):
            h.rivoli_kv_compress_deposit.restype = i
            h.rivoli_kv_compress_deposit.argtypes = [vp] * 6 + [i, i, vp]
            h.rivoli_kv_compress_prefill.restype = i
            h.rivoli_kv_compress_prefill.argtypes = [vp] * 5 + [i, vp]
            h.rivoli_kv_compress_decode.restype = i
            h.rivoli_kv_compress_decode.argtypes = [vp] * 4 + [i, vp]
        if hasattr(h, "rivoli_index_score_blocks"):
            h.rivoli_act_quant_f4_rotated.restype = i
            h.rivoli_act_quant_f4_rotated.argtypes = [vp, i, i, vp]
            h.rivoli_index_score_blocks.restype = i
            h.rivoli_index_score_blocks.argtypes = [vp] * 4 + [i] * 4 + [vp]
        h.rivoli_hash_rows.restype = i
        h.rivoli_hash_rows.argtypes = [vp, i, i, C.c_ulonglong, vp, vp]
        _REF = h
    return _REF
