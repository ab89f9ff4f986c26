"""The entry point that allocates nothing (pto_sfa_quant_launch_static), called through the C ABI with
ctypes: its output must equal that of pto_sfa_quant_launch bit for bit, on two calls in a row, the
second on a smaller input (the built-in scratch array keeps the first call's contents)."""
import ctypes
import os

import pytest
import torch

from pypto_amd.synthetic import gen_sfa_inputs

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "pypto_amd", "libpypto_amd_sfa.so")


class PtoSfaQuantArgs(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in
                ("query_nope", "query_rope", "key_nope_2d", "key_rope_2d", "k_nope_scales", "topk_indices", "block_table",
                 "kv_act_seqs", "attention_out", "workspace")] + \
               [("workspace_bytes", ctypes.c_size_t)] + \
               [(n, ctypes.c_int64) for n in
                ("b", "s1", "nq", "n_kv", "topk", "block_size", "max_blocknum_perbatch", "kv_rows")] + \
               [("softmax_scale", ctypes.c_float), ("num_splits", ctypes.c_int32)]


def _args(d, out, inp, num_splits):
    a = PtoSfaQuantArgs()
    qn, qr, kn, kr, ks, ti, bt, act = d.operator_tensors()
    a.query_nope, a.query_rope = qn.data_ptr(), qr.data_ptr()
    a.key_nope_2d, a.key_rope_2d, a.k_nope_scales = kn.data_ptr(), kr.data_ptr(), ks.data_ptr()
    a.topk_indices, a.block_table, a.kv_act_seqs = ti.data_ptr(), bt.data_ptr(), act.data_ptr()
    a.attention_out = out.data_ptr()
    a.workspace, a.workspace_bytes = None, 0
    a.b, a.s1, a.nq, a.n_kv, a.topk = inp.b, inp.s1, inp.n_q, 1, inp.topk
    a.block_size, a.max_blocknum_perbatch, a.kv_rows = inp.block_size, bt.shape[1], kn.shape[0]
    a.softmax_scale, a.num_splits = inp.softmax_scale, num_splits
    return a


def _both(lib, inp, num_splits):
    dev = torch.device("cuda:0")
    d = inp.to(dev)
    outs = []
    for static in (False, True):
        out = torch.full([inp.b, inp.s1, inp.n_q, 512], float("nan"), dtype=torch.bfloat16, device=dev)
        a = _args(d, out, inp, num_splits)
        if static:
            rc = lib.pto_sfa_quant_launch_static(ctypes.byref(a), None)
        else:
            n = ctypes.c_size_t(0)
            assert lib.pto_sfa_quant_workspace_bytes(ctypes.byref(a), ctypes.byref(n)) == 0
            ws = torch.empty(max(n.value, 16), dtype=torch.uint8, device=dev)
            a.workspace, a.workspace_bytes = ws.data_ptr(), n.value
            rc = lib.pto_sfa_quant_launch(ctypes.byref(a), None)
        assert rc == 0, lib.pto_last_error()
        torch.cuda.synchronize()
        outs.append(out.cpu())
    return outs


def test_static_scratch_entry_point_matches_the_workspace_one():
    lib = ctypes.CDLL(LIB)
    lib.pto_last_error.restype = ctypes.c_char_p
    torch.cuda.synchronize()                                # a context exists; the null stream below is torch's default
    # first call: 6 rows x 128 heads, top-k 1024, four key splits; second call: fewer rows, shorter, two splits
    big = gen_sfa_inputs(3, 2, 128, [5000, 1300, 2600], topk=1024, seed=11)
    small = gen_sfa_inputs(2, 1, 128, [700, 333], topk=256, seed=12)
    for what, inp, ns in (("first", big, 4), ("second, smaller", small, 2)):
        print(f"static scratch, {what} call: b={inp.b} s1={inp.s1} topk={inp.topk} splits={ns}", flush=True)
        ws_out, static_out = _both(lib, inp, ns)
        assert not torch.isnan(static_out).any()
        assert torch.equal(ws_out.view(torch.int16), static_out.view(torch.int16)), what
    # a shape whose splits do not fit the built-in array is refused, with a message, before any launch
    huge = PtoSfaQuantArgs()
    for f in ("query_nope", "query_rope", "key_nope_2d", "key_rope_2d", "k_nope_scales", "topk_indices", "block_table",
              "kv_act_seqs", "attention_out"):
        setattr(huge, f, 256)                               # never dereferenced: the size check comes first
    huge.b, huge.s1, huge.nq, huge.n_kv, huge.topk = 1024, 1, 128, 1, 2048
    huge.block_size, huge.max_blocknum_perbatch, huge.kv_rows = 128, 16, 2048
    huge.softmax_scale, huge.num_splits = 0.04, 8
    assert lib.pto_sfa_quant_launch_static(ctypes.byref(huge), None) == -2
    assert b"scratch" in lib.pto_last_error()


def test_static_scratch_entry_point_with_the_library_s_own_split_choice():
    """num_splits = 0 on a launch of more rows than compute units (300 rows: the first 256 whole, the other 44 in
    five pieces each, partial results in the built-in array): the bits of the workspace entry point with the same
    choice.  When even the fewest splits a shape allows (top-k past what one workgroup holds) exceed the array,
    the call is refused."""
    lib = ctypes.CDLL(LIB)
    lib.pto_last_error.restype = ctypes.c_char_p
    torch.cuda.synchronize()
    inp = gen_sfa_inputs(300, 1, 128, [2048 + 16 * (i % 5) for i in range(300)], topk=2048, seed=13)
    ws_out, static_out = _both(lib, inp, 0)
    assert not torch.isnan(static_out).any()
    assert torch.equal(ws_out.view(torch.int16), static_out.view(torch.int16))
    # top-k 8192 needs four splits at least (2048 keys per workgroup): 128 rows x 4 x 128 heads exceed the array
    forced = PtoSfaQuantArgs()
    for f in ("query_nope", "query_rope", "key_nope_2d", "key_rope_2d", "k_nope_scales", "topk_indices", "block_table",
              "kv_act_seqs", "attention_out"):
        setattr(forced, f, 256)                             # never dereferenced: the size check comes first
    forced.b, forced.s1, forced.nq, forced.n_kv, forced.topk = 128, 1, 128, 1, 8192
    forced.block_size, forced.max_blocknum_perbatch, forced.kv_rows = 128, 64, 8192
    forced.softmax_scale, forced.num_splits = 0.04, 0
    assert lib.pto_sfa_quant_launch_static(ctypes.byref(forced), None) == -2
    assert b"scratch" in lib.pto_last_error()
