"""ctypes loader for the scalar C statement of the goldens (``oracle_c.c``).

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_c.so")
_lib = None

_DT = {torch.float16: 0, torch.float32: 1, torch.bfloat16: 2}


def build(force: bool = False) -> str:
    """Compile oracle_c.c with the Makefile beside it."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-C", _HERE, "liboracle_c.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        _lib.oracle_f32_to_bf16.restype = ctypes.c_uint16
        _lib.oracle_f32_to_fp16.argtypes = [ctypes.c_float]
        _lib.oracle_f32_to_fp16.restype = ctypes.c_uint16
        _lib.oracle_fp16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.oracle_fp16_to_f32.restype = ctypes.c_float
        _lib.oracle_set_threads.argtypes = [ctypes.c_int]
        _lib.oracle_get_threads.restype = ctypes.c_int
        _lib.oracle_sfa_quant.restype = ctypes.c_int
        _lib.oracle_li_decode.restype = ctypes.c_int
    return _lib


def _p(t: torch.Tensor):
    assert t.is_contiguous() and t.device.type == "cpu"
    return ctypes.c_void_p(t.data_ptr())


def set_threads(n: int) -> None:
    lib().oracle_set_threads(int(n))


def get_threads() -> int:
    return int(lib().oracle_get_threads())


def sfa_quant(q_nope, q_rope, kn, kr, kn_scales, topk_indices, block_table, act_seq, b, s1, n, topk,
              block_size, scalar, s2_tile: int = 0) -> torch.Tensor:
    """C golden; tensors as the operator takes them (2-D flattened q, int32 act_seq tensor).
    Returns [b, s1, n, dn] bf16."""
    dn, dr = q_nope.shape[1], q_rope.shape[1]
    out = torch.empty([b, s1, n, dn], dtype=torch.bfloat16)
    act = act_seq.to(torch.int32).contiguous()
    ti = topk_indices.reshape(b * s1, topk).to(torch.int32).contiguous()
    bt = block_table.to(torch.int32).contiguous()
    rc = lib().oracle_sfa_quant(_p(q_nope), _p(q_rope), _p(kn), _p(kr), _p(kn_scales), _p(ti), _p(bt), _p(act),
                                _p(out), ctypes.c_int(b), ctypes.c_int(s1), ctypes.c_int(n), ctypes.c_int(dn),
                                ctypes.c_int(dr), ctypes.c_int(topk), ctypes.c_int(block_size),
                                ctypes.c_int(bt.shape[1]), ctypes.c_float(scalar), ctypes.c_int(s2_tile))
    if rc != 0:
        raise RuntimeError(f"oracle_sfa_quant failed rc={rc}")
    return out


def li_decode(idx_query, idx_query_scale, idx_key_cache, idx_key_scale, idx_weight, act_seq_key, block_table,
              selected_count: int = 2048, return_scores: bool = False):
    """C golden of the indexer.  Returns topk_res [T,1,k] int32 (and scores [T, max_seq] fp32)."""
    t_tot, h, d = idx_query.shape
    act = act_seq_key.to(torch.int32).contiguous()
    b = act.shape[0]
    s1 = t_tot // b
    bs = idx_key_cache.shape[1]
    bt = block_table.to(torch.int32).contiguous()
    res = torch.empty([t_tot, 1, selected_count], dtype=torch.int32)
    stride = max(int(act.max().item()), 1)
    scores = torch.full([t_tot, stride], float("nan"), dtype=torch.float32) if return_scores else None
    qs = idx_query_scale.reshape(t_tot, h).contiguous()
    w = idx_weight.reshape(t_tot, h).contiguous()
    ks = idx_key_scale.reshape(-1).contiguous()
    kc = idx_key_cache.reshape(-1, d).contiguous()
    rc = lib().oracle_li_decode(_p(idx_query.contiguous()), _p(qs), ctypes.c_int(_DT[qs.dtype]), _p(kc), _p(ks),
                                ctypes.c_int(_DT[ks.dtype]), _p(w), ctypes.c_int(_DT[w.dtype]), _p(act), _p(bt),
                                _p(res), _p(scores) if return_scores else ctypes.c_void_p(0),
                                ctypes.c_int64(stride), ctypes.c_int(b), ctypes.c_int(s1), ctypes.c_int(h),
                                ctypes.c_int(d), ctypes.c_int(bs), ctypes.c_int(bt.shape[1]),
                                ctypes.c_int(selected_count))
    if rc != 0:
        raise RuntimeError(f"oracle_li_decode failed rc={rc}")
    return (res, scores) if return_scores else res
