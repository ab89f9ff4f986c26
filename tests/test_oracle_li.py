"""Pins the lightning-indexer oracle (oracle/li_oracle.py, oracle/oracle_c.c).

Independent checks: Python-integer dot products, an integer-arithmetic fp16
rounding, exact rational emulation of the fp32 multiply/add chain, a brute-force
``sorted`` for the select, the second (scalar C) statement, and a set-wise
comparison with a plain torch.bmm / torch.topk evaluation at the reference's own
tolerance.
"""
import struct
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import li_oracle as lo
from pypto_amd.synthetic import gen_indexer_inputs
from pypto_amd.utils import topk_idx_compare


def _f32(x) -> float:
    return struct.unpack("<f", struct.pack("<f", x))[0]


def _rn32(fr: Fraction) -> float:
    """Exact rational -> nearest fp32 (ties to even), integer arithmetic only. Normal range."""
    if fr == 0:
        return 0.0
    sign = -1 if fr < 0 else 1
    fr = abs(fr)
    e = 0
    while fr >= 2:
        fr /= 2
        e += 1
    while fr < 1:
        fr *= 2
        e -= 1
    scaled = fr * (1 << 23)                 # in [2^23, 2^24)
    q, r = divmod(scaled.numerator, scaled.denominator)
    twice = 2 * r
    if twice > scaled.denominator or (twice == scaled.denominator and (q & 1)):
        q += 1
    return sign * float(Fraction(q, 1 << 23) * (Fraction(2) ** e))


def _fp16_round_int(r: int) -> float:
    """float(fp16_rne(r / 2048)) for an integer 0 <= r < 2**21, integers only: keep 11 significant bits."""
    if r == 0:
        return 0.0
    nbits = r.bit_length()
    if nbits <= 11:
        return r / 2048.0
    sh = nbits - 11
    q, rem = r >> sh, r & ((1 << sh) - 1)
    half = 1 << (sh - 1)
    if rem > half or (rem == half and (q & 1)):
        q += 1
    return (q << sh) / 2048.0


def test_dot_is_exact_integer_arithmetic():
    g = torch.Generator().manual_seed(0)
    q = torch.randint(-127, 128, [5, 128], generator=g, dtype=torch.int8)
    k = torch.randint(-127, 128, [9, 128], generator=g, dtype=torch.int8)
    q[0] = 127
    k[0] = 127            # the largest possible dot, 127*127*128
    q[1] = -127
    x = lo.qk_relu_fp16(q.numpy(), k.numpy())
    for h in range(5):
        for j in range(9):
            dot = sum(int(a) * int(b) for a, b in zip(q[h].tolist(), k[j].tolist()))
            assert x[h, j] == _fp16_round_int(max(dot, 0)), (h, j, dot)


def test_relu_scale_fp16_rounding_on_a_grid(c_oracle):
    vals = list(range(0, 5000)) + list(range(2 ** 21 - 5000, 2 ** 21)) + [2 ** k + d for k in range(11, 21)
                                                                              for d in (-3, -2, -1, 0, 1, 2, 3)] \
        + [3 * 2 ** k + d * 2 ** (k - 10) // 2 for k in range(11, 19) for d in range(-4, 5)]
    lib = c_oracle.lib()
    for r in vals:
        want = _fp16_round_int(r)
        got_np = float(np.float32(np.float16(np.float32(r) * np.float32(1 / 2048))))
        got_c = lib.oracle_fp16_to_f32(lib.oracle_f32_to_fp16(r / 2048.0))
        assert got_np == want and got_c == want, r


def test_c_fp16_helpers_roundtrip_all_halves(c_oracle):
    lib = c_oracle.lib()
    halves = np.arange(0, 0x7C00, dtype=np.uint16)             # all non-negative finite fp16
    as_f32 = halves.view(np.float16).astype(np.float32)
    for h, f in zip(halves[::7].tolist(), as_f32[::7].tolist()):
        assert lib.oracle_fp16_to_f32(h) == f
        assert lib.oracle_f32_to_fp16(f) == h
    # ties and near-ties between neighbouring halves, incl. the subnormal range
    for h in [0, 1, 2, 0x3FF, 0x400, 0x401, 0x3C00, 0x7BFE]:
        a, b = float(as_f32[h]), float(as_f32[h + 1])
        mid = (a + b) / 2
        assert lib.oracle_f32_to_fp16(mid) == (h if h % 2 == 0 else h + 1)
        assert lib.oracle_f32_to_fp16(np.nextafter(np.float32(mid), np.float32(b))) == h + 1
        assert lib.oracle_f32_to_fp16(np.nextafter(np.float32(mid), np.float32(a))) == h


def test_head_sum_is_the_stated_fp32_chain():
    g = torch.Generator().manual_seed(1)
    w = (torch.randn(64, generator=g) / 8).to(torch.float32).numpy()
    x = (torch.rand(64, 7, generator=g) * 100).to(torch.float16).to(torch.float32).numpy()
    got = lo.head_sum(w, x)
    for j in range(7):
        acc = 0.0
        for h in range(64):
            prod = _rn32(Fraction(float(w[h])) * Fraction(float(x[h, j])))
            acc = _rn32(Fraction(acc) + Fraction(prod))
        assert float(got[j]) == acc
    # order matters, and the stated order is h ascending
    w2 = np.array([1.0, 2.0 ** -24, 2.0 ** -24, -1.0], dtype=np.float32)
    x2 = np.ones((4, 1), dtype=np.float32)
    assert float(lo.head_sum(w2, x2)[0]) == 0.0
    assert float(lo.head_sum(w2[::-1].copy(), x2)[0]) != 0.0


def test_w_scale_rule_for_both_dtype_families():
    qs = torch.tensor([[0.0123, 0.5]], dtype=torch.float16)
    w = torch.tensor([[0.337, -1.7]], dtype=torch.float16)
    got = lo.w_scale_of(qs, w)
    for i in range(2):
        exact = Fraction(float(qs[0, i])) * Fraction(float(w[0, i]))
        assert float(got[0, i]) == float(np.float16(float(exact)))       # one fp16 rounding of the exact product
    qs32 = torch.tensor([[0.0123, 0.5]], dtype=torch.float32)
    wbf = torch.tensor([[0.337, -1.7]], dtype=torch.bfloat16)
    got = lo.w_scale_of(qs32, wbf)
    for i in range(2):
        exact = Fraction(float(qs32[0, i])) * Fraction(float(wbf[0, i]))
        assert float(got[0, i]) == _rn32(exact)


def _brute_topk(score, eff, k):
    n = max(min(eff, len(score)), 0)
    order = sorted(range(n), key=lambda j: (-float(score[j]) if score[j] != 0 else 0.0, j))
    return (order[:k] + [-1] * k)[:k]


@pytest.mark.parametrize("case", ["random", "ties", "all_equal", "zeros_pm", "short", "exact_k", "k_plus_1",
                                  "negative", "empty"])
def test_canonical_select_against_sorted(case):
    g = np.random.default_rng(3)
    k = 16
    if case == "random":
        s, eff = g.standard_normal(100).astype(np.float32), 100
    elif case == "ties":
        s, eff = g.integers(0, 5, 200).astype(np.float32), 200
    elif case == "all_equal":
        s, eff = np.full(64, 1.5, dtype=np.float32), 64
    elif case == "zeros_pm":
        s = np.array([0.0, -0.0] * 20, dtype=np.float32)
        s[7] = 1.0
        eff = 40
    elif case == "short":
        s, eff = g.standard_normal(100).astype(np.float32), 9
    elif case == "exact_k":
        s, eff = g.integers(0, 3, 100).astype(np.float32), 16
    elif case == "k_plus_1":
        s, eff = g.integers(0, 3, 100).astype(np.float32), 17
    elif case == "negative":
        s, eff = -np.abs(g.standard_normal(50)).astype(np.float32), 50
    else:
        s, eff = g.standard_normal(10).astype(np.float32), 0
    assert lo.canonical_topk(s, eff, k).tolist() == _brute_topk(s, eff, k)


def _inputs(variant, seed, b=3, s1=2, act=(300, 129, 5), k=64):
    return gen_indexer_inputs(b, s1, list(act), selected_count=k, seed=seed, variant=variant)


@pytest.mark.parametrize("variant", ["fp16", "fp32"])
def test_c_statement_is_bit_identical(c_oracle, variant):
    inp = _inputs(variant, 5)
    ref = lo.lightning_indexer_ref(inp.idx_query, inp.idx_query_scale, inp.idx_key_cache, inp.idx_key_scale,
                                   inp.idx_weight, inp.act_seq_key, inp.block_table, inp.selected_count)
    got, scores = c_oracle.li_decode(inp.idx_query, inp.idx_query_scale, inp.idx_key_cache, inp.idx_key_scale,
                                     inp.idx_weight, inp.act_seq_key, inp.block_table, inp.selected_count,
                                     return_scores=True)
    assert torch.equal(got, ref)
    rows = lo.li_scores(inp.idx_query, inp.idx_query_scale, inp.idx_key_cache, inp.idx_key_scale, inp.idx_weight,
                        inp.act_seq, inp.block_table)
    for t, row in enumerate(rows):
        assert np.array_equal(scores[t, :len(row)].numpy().view(np.uint32), row.view(np.uint32))


def test_causal_effective_length_and_padding():
    inp = _inputs("fp16", 6, b=2, s1=2, act=(40, 1), k=64)
    res = lo.lightning_indexer_ref(inp.idx_query, inp.idx_query_scale, inp.idx_key_cache, inp.idx_key_scale,
                                   inp.idx_weight, inp.act_seq_key, inp.block_table, 64)
    assert int((res[0, 0] >= 0).sum()) == 39 and int((res[1, 0] >= 0).sum()) == 40
    assert 39 not in res[0, 0].tolist() and 39 in res[1, 0].tolist()
    assert torch.all(res[2, 0] == -1)                      # act=1, first of two tokens: nothing visible
    assert res[3, 0, 0] == 0 and torch.all(res[3, 0, 1:] == -1)
    assert sorted(res[1, 0, :40].tolist()) == list(range(40))


def test_setwise_agreement_with_plain_torch_evaluation():
    """torch.bmm + torch.topk (library summation order and tie order) must agree as sets
    within the reference's own tolerance: 0.5 % of a row."""
    inp = gen_indexer_inputs(2, 1, [4096, 3000], selected_count=512, seed=7, variant="fp16")
    ref = lo.lightning_indexer_ref(inp.idx_query, inp.idx_query_scale, inp.idx_key_cache, inp.idx_key_scale,
                                   inp.idx_weight, inp.act_seq_key, inp.block_table, 512)
    key = inp.idx_key_cache.reshape(-1, 128)
    ks = inp.idx_key_scale.reshape(-1).float()
    out = torch.empty_like(ref)
    for b in range(2):
        n = inp.act_seq[b]
        pos = torch.arange(n)
        phys = inp.block_table[b].long()[pos // 128] * 128 + pos % 128
        dot = torch.matmul(inp.idx_query[b].to(torch.int32), key[phys].t().to(torch.int32)).float().relu()
        x = (dot * (1 / 2048)).to(torch.float16).float()
        w = (inp.idx_query_scale[b] * inp.idx_weight[b]).float()
        sc = torch.matmul(w[None], x)[0] * ks[phys]
        out[b, 0] = torch.topk(sc, 512).indices.to(torch.int32)
    topk_idx_compare(out, ref, "topk_res", 5e-3, 512)


def _fp16_rne(x: Fraction) -> float:
    """Exact rational -> nearest fp16, ties to even; handles subnormals; overflow not needed here."""
    if x == 0:
        return 0.0
    sign = -1.0 if x < 0 else 1.0
    x = abs(x)
    e = -14
    while x >= Fraction(2) ** (e + 1):
        e += 1
    unit = Fraction(2) ** (e - 10)                    # spacing of fp16 values in [2^e, 2^(e+1)) (and below 2^-14)
    q, r = divmod(x, unit)
    q = int(q)
    if 2 * r > unit or (2 * r == unit and (q & 1)):
        q += 1
    return sign * float(q * unit)


def test_fp16_dequant_variant_against_exact_rationals():
    """The chained C++ operator's rounding model: every fp16 product and the fp32 head sum restated with
    exact rationals on a small case; and it differs from the operator's own model."""
    inp = gen_indexer_inputs(1, 1, [40], selected_count=8, seed=5, variant="fp16", n_heads=64)
    rows = lo.li_scores_fp16_dequant(inp.idx_query, inp.idx_query_scale, inp.idx_key_cache, inp.idx_key_scale,
                                     inp.idx_weight, inp.act_seq, inp.block_table)
    q = inp.idx_query[0].numpy().astype(int)
    kc = inp.idx_key_cache.reshape(-1, 128).numpy().astype(int)
    ks = inp.idx_key_scale.reshape(-1).numpy()
    qs = inp.idx_query_scale[0].numpy()
    wt = inp.idx_weight[0].numpy()
    bt = inp.block_table[0].numpy()
    for j in (0, 7, 39):
        phys = int(bt[j // 128]) * 128 + j % 128
        acc = 0.0
        for h in range(64):
            dot = int(np.dot(q[h], kc[phys]))
            v = _fp16_rne(Fraction(dot, 2048))
            v = _fp16_rne(Fraction(v) * Fraction(float(qs[h])))
            v = _fp16_rne(Fraction(v) * Fraction(float(ks[phys])))
            v = max(v, 0.0)
            v = _fp16_rne(Fraction(v) * Fraction(float(wt[h])))
            acc = _rn32(Fraction(acc) + Fraction(v))
        assert rows[0][j] == np.float32(acc), (j, rows[0][j], acc)
    other = lo.li_scores(inp.idx_query, inp.idx_query_scale, inp.idx_key_cache, inp.idx_key_scale, inp.idx_weight,
                         inp.act_seq, inp.block_table)
    assert not np.array_equal(other[0], rows[0])
    # same ranking up to near-ties: the two models select almost the same keys
    a = set(lo.canonical_topk(rows[0], 40, 8).tolist())
    b = set(lo.canonical_topk(other[0], 40, 8).tolist())
    assert len(a & b) >= 6
