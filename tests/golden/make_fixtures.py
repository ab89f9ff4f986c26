#!/usr/bin/env python3
"""Writes the golden fixtures of this directory: small seeded inputs of both operators together with
the outputs of the CPU goldens (oracle/sfa_oracle.py, oracle/li_oracle.py) for them.

    python tests/golden/make_fixtures.py

The fixtures freeze inputs AND expected outputs, so that a later change of a generator or of a golden
shows up as a failing test (tests/test_golden_fixtures.py) instead of silently moving the bar.  They
are plain numpy archives (bf16 / fp16 tensors stored as their 16-bit patterns), loaded with
allow_pickle=False.  The reference holds no stored vectors for this path; its own drivers generate
inputs and goldens at run time (deepseekv32_sparse_flash_attention_quant.py:298-388,
deepseekv32_lightning_indexer_quant.py:119-181), which is what these files stand in for.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle import li_oracle, sfa_oracle  # noqa: E402
from pypto_amd.synthetic import gen_indexer_inputs, gen_sfa_inputs  # noqa: E402


def bits(t: torch.Tensor) -> np.ndarray:
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.contiguous().view(torch.int16).numpy()
    return t.contiguous().numpy()


def sfa_fixture():
    inp = gen_sfa_inputs(2, 2, 16, [200, 40], topk=64, seed=11)
    args = (inp.q_bsnd(), inp.key_nope_2d, inp.key_rope_2d, inp.k_nope_scales, inp.topk_indices, inp.block_table,
            inp.actual_seq, inp.block_size, inp.softmax_scale, inp.topk)
    single = sfa_oracle.sfa_single_pass(*args)
    online = sfa_oracle.sfa_online(*args, s2_tile=32)
    np.savez_compressed(
        os.path.join(HERE, "sfa_b2_s2_h16_topk64.npz"),
        query_nope_bf16=bits(inp.query_nope), query_rope_bf16=bits(inp.query_rope), key_nope_2d=bits(inp.key_nope_2d),
        key_rope_2d_bf16=bits(inp.key_rope_2d), k_nope_scales=bits(inp.k_nope_scales),
        topk_indices=bits(inp.topk_indices), block_table=bits(inp.block_table), kv_act_seqs=bits(inp.kv_act_seqs),
        softmax_scale=np.float32(inp.softmax_scale), block_size=np.int32(inp.block_size), topk=np.int32(inp.topk),
        n_q=np.int32(inp.n_q), out_single_pass_bf16=bits(single), out_online_tile32_bf16=bits(online))


def li_fixture():
    for variant in ("fp16", "fp32"):
        inp = gen_indexer_inputs(2, 2, [300, 40], selected_count=16, seed=12, variant=variant)
        res = li_oracle.lightning_indexer_ref(inp.idx_query, inp.idx_query_scale, inp.idx_key_cache, inp.idx_key_scale,
                                              inp.idx_weight, inp.act_seq_key, inp.block_table, inp.selected_count)
        np.savez_compressed(
            os.path.join(HERE, f"li_b2_s2_k16_{variant}.npz"),
            idx_query=bits(inp.idx_query), idx_query_scale=bits(inp.idx_query_scale),
            idx_key_cache=bits(inp.idx_key_cache), idx_key_scale=bits(inp.idx_key_scale),
            idx_weight=bits(inp.idx_weight), act_seq_key=bits(inp.act_seq_key), block_table=bits(inp.block_table),
            selected_count=np.int32(inp.selected_count), topk_res=bits(res))


if __name__ == "__main__":
    sfa_fixture()
    li_fixture()
    print("fixtures written to", HERE)
