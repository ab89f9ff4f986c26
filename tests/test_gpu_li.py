"""Parity of the HIP lightning indexer (through the operator, pybind11 and the C ABI) against the CPU
oracle.  The bar is bit-exact indices."""
import numpy as np
import pytest
import torch

import pypto_amd
from pypto_amd.synthetic import gen_indexer_inputs

pytestmark = pytest.mark.gpu


def run_op(inp):
    dev = torch.device("cuda:0")
    d = inp.to(dev)
    d.topk_res.fill_(-7)
    ts = [pypto_amd.from_torch(t) for t in d.operator_tensors()]
    ret = pypto_amd.lightning_indexer_decode(*ts, [128, 64, 32, 16, 8, 4, 1], pypto_amd.LightningIndexerConfigs(),
                                             inp.selected_count)
    assert ret is None
    torch.cuda.synchronize()
    return d.topk_res.cpu()


def oracle(inp, c_oracle):
    return c_oracle.li_decode(inp.idx_query, inp.idx_query_scale, inp.idx_key_cache, inp.idx_key_scale,
                              inp.idx_weight, inp.act_seq_key, inp.block_table, inp.selected_count)


def assert_exact(got, ref, what):
    if not torch.equal(got, ref):
        bad = (got != ref).reshape(got.shape[0], -1)
        rows = torch.nonzero(bad.any(dim=1)).reshape(-1).tolist()
        r = rows[0]
        cols = torch.nonzero(bad[r]).reshape(-1)[:8].tolist()
        raise AssertionError(f"{what}: {int(bad.sum())} index mismatches in rows {rows[:8]}; row {r} cols {cols}: "
                             f"got {got[r, 0, cols].tolist()} want {ref[r, 0, cols].tolist()}")


@pytest.mark.parametrize("variant", ["fp16", "fp32"])
@pytest.mark.parametrize("b,s1,act,k", [
    (2, 1, [4096, 3000], 2048),        # above the select threshold, one ragged
    (3, 2, [300, 129, 5], 64),         # two query tokens per sequence, causal effective lengths
    (2, 1, [2048, 2049], 2048),        # exactly k and k+1 candidates
    (2, 1, [100, 1], 2048),            # fewer candidates than k: padded with -1
    (1, 4, [9000], 2048),              # s1 = 4
    (1, 1, [33], 16),                  # partial 32-key block
    # the two shapes of the reference's own system tests
    # (framework/tests/st/operator/src/test_deepseek_v3.2_exp/gen_lightning_indexer.py:374-376, 428-430)
    (4, 1, [768, 4097, 8192, 131071], 2048),
    (4, 2, [65536] * 4, 2048),
])
def test_indexer_bit_exact(c_oracle, variant, b, s1, act, k):
    inp = gen_indexer_inputs(b, s1, act, selected_count=k, seed=7 * b + s1 + k, variant=variant)
    assert_exact(run_op(inp), oracle(inp, c_oracle), f"{variant} b={b} s1={s1} act={act} k={k}")


def test_engineered_ties_and_zero_scores(c_oracle):
    """Many equal scores: zero weights make every score +-0, duplicated key rows make exact ties."""
    inp = gen_indexer_inputs(2, 1, [5000, 6000], selected_count=2048, seed=31, variant="fp16")
    inp.idx_weight[0] = 0                                # token 0: all scores are zero -> positions 0..2047
    kc = inp.idx_key_cache.reshape(-1, 128)
    ks = inp.idx_key_scale.reshape(-1)
    # token 1: every logical position p >= 3000 repeats the row of position p - 3000
    pos = torch.arange(6000)
    phys = inp.block_table[1].long()[pos // 128] * 128 + pos % 128
    kc[phys[3000:]] = kc[phys[:3000]]
    ks[phys[3000:]] = ks[phys[:3000]]
    got = run_op(inp)
    ref = oracle(inp, c_oracle)
    assert ref[0, 0].tolist() == list(range(2048))
    assert_exact(got, ref, "ties")


def test_negative_weights_and_mixed_signs(c_oracle):
    inp = gen_indexer_inputs(1, 1, [7000], selected_count=2048, seed=41, variant="fp32")
    inp.idx_weight[:] = -inp.idx_weight.abs()            # all scores <= 0: the best are the zeros
    assert_exact(run_op(inp), oracle(inp, c_oracle), "negative")


def test_config1_full_size(c_oracle):
    """B=4, KV 32768 each, shuffled block table, top-2048."""
    for variant in ("fp16", "fp32"):
        inp = gen_indexer_inputs(4, 1, [32768] * 4, selected_count=2048, seed=1, variant=variant)
        assert_exact(run_op(inp), oracle(inp, c_oracle), f"cfg1 {variant}")


def test_bf16_key_scales(c_oracle):
    """Key scales in bf16 (two per staged dword, either half), fp16 query scales, bf16 weights."""
    inp = gen_indexer_inputs(2, 2, [4500, 2600], selected_count=2048, seed=51, variant="fp32")
    inp.idx_key_scale = inp.idx_key_scale.to(torch.bfloat16)
    inp.idx_query_scale = inp.idx_query_scale.to(torch.float16)
    assert_exact(run_op(inp), oracle(inp, c_oracle), "bf16 key scales")


def test_long_runs_wide_block_table(c_oracle):
    """64 query tokens over a block table 1024 pages wide: the launch then gives every wave the longest
    run of keys it supports, the lengths end inside runs, pairs and 32-key blocks, and the longest
    sequence is the maximum the operator accepts (131072)."""
    from pypto_amd.synthetic import gen_block_table
    g = torch.Generator().manual_seed(61)
    act = [131072, 65536 + 17, 40000, 2049, 2048, 2047, 4096 + 33, 1] + \
          [int(x) for x in torch.randint(1, 3000, [56], generator=g)]
    block_num, table = gen_block_table(act, 128, g, shuffle=True, max_kv=131072)
    inp = gen_indexer_inputs(len(act), 1, act, selected_count=2048, seed=62, variant="fp32", block_table=table,
                             block_num=block_num)
    assert_exact(run_op(inp), oracle(inp, c_oracle), "wide block table")


@pytest.mark.parametrize("b,s1", [
    (100, 1),     # balanced run mapping, rows 1.. of the token table (tokens 64 and up)
    (40, 4),      # the same with four query tokens per sequence
    (130, 4),     # 520 tokens: past the balanced mapping, one grid row per token
])
def test_many_query_tokens_short_sequences(c_oracle, b, s1):
    """More query tokens than one row of the score kernel's token table holds, and more than the balanced
    mapping takes at all; short ragged sequences so the oracle stays cheap."""
    g = torch.Generator().manual_seed(1000 + b)
    act = [int(x) for x in torch.randint(s1, 700, [b], generator=g)]
    act[0], act[-1] = 699, s1                      # a long first and the shortest possible last sequence
    inp = gen_indexer_inputs(b, s1, act, selected_count=128, seed=b + s1, variant="fp16")
    assert_exact(run_op(inp), oracle(inp, c_oracle), f"b={b} s1={s1}")


@pytest.mark.parametrize("variant,b,s1", [("fp32", 28, 3), ("fp16", 28, 4)])
def test_token_pairs_share_a_key_pass(c_oracle, variant, b, s1):
    """Enough work for the launch to score two query tokens of a sequence per key pass (the reference scores
    all s1 tokens against a page at once, lightning_indexer_quant_impl.py:163-169): an odd s1 leaves a unit of
    one token, s1 = 4 makes two units per sequence; ragged lengths end inside runs and pairs."""
    g = torch.Generator().manual_seed(300 + b)
    act = [int(x) for x in torch.randint(2100, 20480, [b], generator=g)]
    act[0], act[1] = 20480, 2049
    inp = gen_indexer_inputs(b, s1, act, selected_count=2048, seed=b * s1, variant=variant)
    assert inp.b * ((s1 + 1) // 2) * (inp.block_table.shape[1] * 128 // 64) >= 8 * 256 * 8, "shape too small for token pairs"
    assert_exact(run_op(inp), oracle(inp, c_oracle), f"{variant} b={b} s1={s1}")


@pytest.mark.parametrize("variant,b,s1", [("fp16", 260, 4), ("fp32", 260, 3)])
def test_token_pairs_beyond_the_balanced_mapping(c_oracle, variant, b, s1):
    """Token pairs per key pass in the launch shape that takes one grid row per unit: more than 512 units (260
    sequences of two units each) with enough keys for the pair form -- the far end of the operator's documented
    decode range (b up to 128 with s1 up to 4 and long KV, examples/models/deepseek_v32_exp/README.md:6-24, and
    past it).  The odd s1 leaves every sequence a unit of one token."""
    g = torch.Generator().manual_seed(500 + s1)
    act = [int(x) for x in torch.randint(s1, 2300, [b], generator=g)]
    act[0], act[1], act[-1] = 2300, 2049, s1
    inp = gen_indexer_inputs(b, s1, act, selected_count=2048, seed=b + s1, variant=variant)
    units = inp.b * ((s1 + 1) // 2)
    assert units > 512, "shape must be past the balanced mapping"
    assert units * (inp.block_table.shape[1] * 128 // 64) >= 8 * 256 * 8, "shape too small for token pairs"
    assert_exact(run_op(inp), oracle(inp, c_oracle), f"{variant} b={b} s1={s1}")


def test_small_pages_and_small_k(c_oracle):
    """32-key pages (every block of a pair on its own page) and small selection counts."""
    for k, act in ((1, [5000, 70]), (17, [2500, 31]), (512, [700, 513])):
        inp = gen_indexer_inputs(2, 1, act, selected_count=k, seed=70 + k, variant="fp16", block_size=32)
        assert_exact(run_op(inp), oracle(inp, c_oracle), f"bs=32 k={k}")


def test_select_falls_back_on_degenerate_rows(c_oracle):
    """Rows the sampled pivot cannot split: a constant row with one spike (every sampled score equal),
    and two-valued scores where far more than the list holds tie above the pivot."""
    inp = gen_indexer_inputs(2, 1, [40000, 30000], selected_count=2048, seed=81, variant="fp32")
    kc = inp.idx_key_cache.reshape(-1, 128)
    ks = inp.idx_key_scale.reshape(-1)
    pos0 = torch.arange(40000)
    phys0 = inp.block_table[0].long()[pos0 // 128] * 128 + pos0 % 128
    kc[phys0] = kc[phys0[0]].clone()              # token 0: every key equal ...
    ks[phys0] = ks[phys0[0]].clone()
    ks[phys0[12345]] = ks[phys0[0]].clone() * 4   # ... except one, four times the score
    pos1 = torch.arange(30000)
    phys1 = inp.block_table[1].long()[pos1 // 128] * 128 + pos1 % 128
    kc[phys1] = kc[phys1[0]].clone()              # token 1: two score values, 3/4 of the keys on the larger
    ks[phys1] = ks[phys1[0]].clone()
    ks[phys1[pos1 % 4 == 1]] = ks[phys1[0]].clone() * 0.5
    assert_exact(run_op(inp), oracle(inp, c_oracle), "degenerate rows")


def run_variant(inp):
    dev = torch.device("cuda:0")
    d = inp.to(dev)
    d.topk_res.fill_(-7)
    ret = pypto_amd.lightning_indexer_decode(*d.operator_tensors(), None, None, inp.selected_count,
                                             arith_variant="fp16_dequant")
    assert ret is None
    torch.cuda.synchronize()
    return d.topk_res.cpu()


@pytest.mark.parametrize("b,s1,act,k", [
    (2, 1, [4096, 3000], 2048),
    (3, 2, [300, 129, 5], 64),
    (1, 1, [33], 16),
    (2, 2, [9000, 2049], 2048),
])
def test_fp16_dequant_variant_bit_exact(b, s1, act, k):
    """The arithmetic of the reference's chained C++ operator (fp16 scales applied before the ReLU), against
    its own oracle."""
    from oracle import li_oracle as lo
    inp = gen_indexer_inputs(b, s1, act, selected_count=k, seed=11 * b + s1 + k, variant="fp16")
    want = lo.lightning_indexer_fp16_dequant_ref(inp.idx_query, inp.idx_query_scale, inp.idx_key_cache, inp.idx_key_scale,
                                                 inp.idx_weight, inp.act_seq_key, inp.block_table, k)
    assert_exact(run_variant(inp), want, f"fp16_dequant b={b} s1={s1} act={act} k={k}")


def test_fp16_dequant_variant_refuses_other_dtypes():
    inp = gen_indexer_inputs(1, 1, [300], selected_count=64, seed=1, variant="fp32").to(torch.device("cuda:0"))
    with pytest.raises(TypeError):
        pypto_amd.lightning_indexer_decode(*inp.operator_tensors(), None, None, 64, arith_variant="fp16_dequant")
    with pytest.raises(ValueError):
        pypto_amd.lightning_indexer_decode(*inp.operator_tensors(), None, None, 64, arith_variant="other")
