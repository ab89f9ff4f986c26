"""Pins the indexer-prolog oracle (oracle/lip_oracle.py).

Independent checks: Python-integer matmul, an integer-arithmetic bf16 rounding, exact rational
emulation of the fp32 sums (order included), float64 statistics for the layer norm, rotation
identities for rope, known answers for the int8 quantisation, and the whole function against
the golden's statements evaluated with torch's own matmul/mean at the reference's tolerances
(examples/models/deepseek_v32_exp/deepseekv32_lightning_indexer_prolog_quant.py:424-428).
"""
import struct
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import lip_oracle as lo
from pypto_amd.synthetic import gen_indexer_prolog_inputs


def _rn32(fr: Fraction) -> float:
    """Exact rational -> nearest fp32 (ties to even); normal range."""
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
    scaled = fr * (1 << 23)
    q, r = divmod(scaled.numerator, scaled.denominator)
    if 2 * r > scaled.denominator or (2 * r == scaled.denominator and (q & 1)):
        q += 1
    return sign * float(Fraction(q, 1 << 23) * (Fraction(2) ** e))


def _bf16_int(x: float) -> float:
    """fp32 -> bf16 ties-to-even through the bit pattern, scalar integer arithmetic."""
    (u,) = struct.unpack("<I", struct.pack("<f", x))
    low = u & 0xFFFF
    u >>= 16
    if low > 0x8000 or (low == 0x8000 and (u & 1)):
        u += 1
    return struct.unpack("<f", struct.pack("<I", (u << 16) & 0xFFFFFFFF))[0]


def _bf16_vals(rng, shape, scale=1.0):
    return lo.bf16_round((rng.standard_normal(shape) * scale).astype(np.float32))


def test_bf16_round_matches_integer_statement():
    rng = np.random.default_rng(0)
    v = np.concatenate([rng.standard_normal(4000).astype(np.float32) * 37,
                        np.array([1.00390625, 1.01171875, 1.0, -1.00390625, 3.0e-5, 65280.0, 0.0], np.float32)])
    # 1.00390625 = 1 + 2**-8: exactly half way between bf16 1.0 and 1.0078125 -> even (1.0)
    got = lo.bf16_round(v)
    exp = np.array([_bf16_int(float(a)) for a in v], np.float32)
    assert np.array_equal(got, exp)
    assert got[4000] == 1.0 and got[4001] == np.float32(1.015625)
    assert np.array_equal(got, torch.from_numpy(v).to(torch.bfloat16).float().numpy())


def test_q_linear_against_python_integers():
    rng = np.random.default_rng(1)
    a = rng.integers(-128, 128, (3, 40), dtype=np.int8)
    w = rng.integers(-128, 128, (40, 5), dtype=np.int8)
    got = lo.q_linear(a, w)
    for t in range(3):
        for n in range(5):
            assert int(got[t, n]) == sum(int(a[t, k]) * int(w[k, n]) for k in range(40))
    # extreme operands stay inside int32
    big = lo.q_linear(np.full((1, 2048), -128, np.int8), np.full((2048, 1), -128, np.int8))
    assert int(big[0, 0]) == 2048 * 128 * 128


def test_blocked_dot_order_exact_rational():
    rng = np.random.default_rng(2)
    x = _bf16_vals(rng, (2, 1152), 50.0)          # 18 blocks: groups of 8, 8 and 2
    w = _bf16_vals(rng, (1152, 2), 50.0)
    got = lo.blocked_dot(x, w)
    for t in range(2):
        for n in range(2):
            total = 0.0
            for g0 in range(0, 18, 8):
                gsum = 0.0
                for c in range(g0, min(g0 + 8, 18)):
                    acc = 0.0
                    for k in range(64 * c, 64 * c + 64):
                        acc = _rn32(Fraction(acc) + Fraction(float(x[t, k])) * Fraction(float(w[k, n])))
                    gsum = _rn32(Fraction(gsum) + Fraction(acc))
                total = _rn32(Fraction(total) + Fraction(gsum))
            assert got[t, n] == np.float32(total)


def test_blocked_dot_is_order_sensitive():
    # 2**24 followed by ones: where the ones meet the big term decides whether they survive
    w = np.ones((1024, 1), np.float32)
    x = np.zeros((1, 1024), np.float32)
    x[0, 0] = 2.0 ** 24
    x[0, 64:128] = 1.0                             # block 1 of group 0
    x[0, 512:] = 1.0                               # group 1
    got = lo.blocked_dot(x, w)
    # block level: 2**24 alone in block 0; block 1 = 64; group 0 = 2**24 + 64; group 1 = 512
    assert got[0, 0] == np.float32(2.0 ** 24 + 64 + 512)
    # a single ascending chain loses every one of them
    assert lo.blocked_dot(x, w, block=1024)[0, 0] == np.float32(2.0 ** 24)
    # the second level matters too: 2**24 in block 0, every later block sums to exactly 1.0.  With groups
    # of eight the seven ones of group 0 are lost one by one but group 1 arrives as 8.0 and survives;
    # one chain over all sixteen block sums loses all fifteen.
    x2 = np.full((1, 1024), 1.0 / 64, np.float32)
    x2[0, :64] = 0.0
    x2[0, 0] = 2.0 ** 24
    assert lo.blocked_dot(x2, w)[0, 0] == np.float32(2.0 ** 24 + 8)
    assert lo.blocked_dot(x2, w, group=16)[0, 0] == np.float32(2.0 ** 24)


def test_pair_tree_sum_order():
    v = np.zeros(128, np.float32)
    v[0] = 2.0 ** 24
    v[1] = 1.0          # lost: added to 2**24 first
    v[2] = v[3] = 1.0   # survive: added to each other first
    assert lo.pair_tree_sum(v) == np.float32(2.0 ** 24 + 2)
    rng = np.random.default_rng(3)
    u = rng.standard_normal((5, 128)).astype(np.float32)
    exp = []
    for row in u:
        cur = [float(a) for a in row]
        while len(cur) > 1:
            cur = [_rn32(Fraction(cur[i]) + Fraction(cur[i + 1])) for i in range(0, len(cur), 2)]
        exp.append(cur[0])
    assert np.array_equal(lo.pair_tree_sum(u), np.array(exp, np.float32))


def test_hadamard_seq_identity_order_and_rational():
    rng = np.random.default_rng(4)
    a = _bf16_vals(rng, (3, 2, 128), 4.0)
    assert np.array_equal(lo.hadamard_seq(a, np.eye(128, dtype=np.float32)), a)
    # a permutation matrix moves channels
    perm = rng.permutation(128)
    p = np.zeros((128, 128), np.float32)
    p[np.arange(128), perm] = 1.0
    out = lo.hadamard_seq(a, p)
    assert np.array_equal(out[..., perm], a)
    # exact rational restatement of the ascending chain
    h = _bf16_vals(rng, (128, 128), 1.0)
    got = lo.hadamard_seq(a[0], h)
    for row in range(2):
        for j in (0, 17, 127):
            acc = 0.0
            for i in range(128):
                acc = _rn32(Fraction(acc) + Fraction(float(a[0, row, i])) * Fraction(float(h[i, j])))
            assert got[row, j] == np.float32(_bf16_int(acc))
    # order matters: big, then many ones (lost one by one)
    v = np.zeros((1, 128), np.float32)
    v[0, 0] = 2.0 ** 24
    v[0, 1:] = 1.0
    ones = np.ones((128, 1), np.float32)
    assert lo.hadamard_seq(v, ones)[0, 0] == np.float32(2.0 ** 24)
    assert lo.hadamard_seq(v[:, ::-1], ones)[0, 0] == lo.bf16_round(np.float32(2.0 ** 24 + 127))


def test_rope_first_rotation_properties():
    rng = np.random.default_rng(5)
    x = _bf16_vals(rng, (4, 3, 128), 2.0)
    zero = np.zeros((4, 64), np.float32)
    one = np.ones((4, 64), np.float32)
    assert np.array_equal(lo.rope_first(x, one, zero), x)                     # angle 0
    q = lo.rope_first(x, zero, one)                                           # angle pi/2: (a, b) -> (-b, a)
    assert np.array_equal(q[..., :32], -x[..., 32:64]) and np.array_equal(q[..., 32:64], x[..., :32])
    assert np.array_equal(q[..., 64:], x[..., 64:])                           # untouched channels
    ang = rng.uniform(0, 2 * np.pi, (4, 64))
    cos = lo.bf16_round(np.cos(ang).astype(np.float32))
    sin = lo.bf16_round(np.sin(ang).astype(np.float32))
    got = lo.rope_first(x, cos, sin).astype(np.float64)
    a, b = x[..., :32].astype(np.float64), x[..., 32:64].astype(np.float64)
    c, s = cos.astype(np.float64)[:, None, :], sin.astype(np.float64)[:, None, :]
    exp = np.concatenate([a * c[..., :32] - b * s[..., :32], b * c[..., 32:] + a * s[..., 32:]], axis=-1)
    assert np.max(np.abs(got[..., :64] - exp)) <= 2.0 ** -8 * np.max(np.abs(exp))   # one bf16 rounding


def test_quant_int8_known_answers():
    y = np.zeros((3, 128), np.float32)
    y[0, 5] = 4.0
    y[0, 6] = -2.0
    y[0, 7] = 0.015625
    y[1, :] = np.linspace(-8, 8, 128, dtype=np.float32)
    q, s = lo.quant_int8(lo.bf16_round(y))
    assert q[0, 5] == 127 and q[0, 6] == -64 and q[0, 7] == 0      # -63.5 -> -64 (ties to even), 0.496 -> 0
    assert s[0] == np.float16(np.float32(1.0) / (np.float32(127.0) / np.float32(4.0)))
    assert q[1, 0] == -127 and q[1, -1] == 127 and abs(float(s[1]) * 127 - 8.0) < 8.0 * 2 ** -10
    assert not q[2].any() and s[2] == 0                              # all-zero row: defined as zeros
    rng = np.random.default_rng(6)
    v = _bf16_vals(rng, (50, 128), 9.0)
    q, s = lo.quant_int8(v)
    assert np.abs(q.astype(np.int32)).max(axis=-1).tolist() == [127] * 50
    assert np.max(np.abs(q.astype(np.float64) * s.astype(np.float64)[:, None] - v)) <= \
        0.51 * s.max() + 2 ** -10 * np.abs(v).max()


def test_layer_norm_against_float64():
    rng = np.random.default_rng(7)
    x = (rng.standard_normal((9, 128)) * 13 + 4).astype(np.float32)
    gamma = _bf16_vals(rng, (128,), 1.0)
    beta = _bf16_vals(rng, (128,), 1.0)
    got = lo.layer_norm_fixed(x, gamma, beta, 1e-6).astype(np.float64)
    xd = x.astype(np.float64)
    mean = xd.mean(-1, keepdims=True)
    var = ((xd - mean) ** 2).mean(-1, keepdims=True)
    exp = (xd - mean) / np.sqrt(var + 1e-6) * gamma + beta
    assert np.max(np.abs(got - exp)) <= 2.0 ** -8 * np.abs(exp).max() + 1e-5
    plain = lo.layer_norm_fixed(x, np.ones(128, np.float32), np.zeros(128, np.float32), 1e-6)
    assert abs(float(plain.mean())) < 2e-3 and abs(float(plain.var()) - 1.0) < 2e-2


def _small(seed, **kw):
    args = dict(b=2, s1=2, act_seq=[300, 129], seed=seed, h=256, q_lora_rank=512, n_heads=4)
    args.update(kw)
    return gen_indexer_prolog_inputs(**args)


def test_scatter_touches_only_named_rows():
    i = _small(11)
    r = lo.indexer_prolog_ref(*i.input_tensors())
    kc0 = i.k_cache.numpy().reshape(-1, 128)
    ks0 = i.k_cache_scale.numpy().reshape(-1)
    kc1 = r["k_cache"].reshape(-1, 128)
    ks1 = r["k_cache_scale"].reshape(-1)
    rows = i.k_cache_index.numpy()
    assert len(set(rows.tolist())) == 4
    mask = np.ones(kc0.shape[0], bool)
    mask[rows] = False
    assert np.array_equal(kc0[mask], kc1[mask]) and np.array_equal(ks0[mask], ks1[mask])
    assert np.array_equal(kc1[rows], r["k_int8"]) and np.array_equal(ks1[rows], r["k_scale"])
    # positions: the last s1 tokens of each sequence through the page table
    table = i.block_table.numpy()
    exp = [table[b, (a - 2 + j) // 128] * 128 + (a - 2 + j) % 128 for b, a in enumerate(i.act_seq) for j in range(2)]
    assert rows.tolist() == exp
    # an index outside the cache is ignored
    bad = i.k_cache_index.clone()
    bad[1] = -1
    bad[2] = kc0.shape[0]
    args = list(i.input_tensors())
    args[15] = bad
    r2 = lo.indexer_prolog_ref(*args)
    kc2 = r2["k_cache"].reshape(-1, 128)
    assert np.array_equal(kc2[rows[1]], kc0[rows[1]]) and np.array_equal(kc2[rows[2]], kc0[rows[2]])
    assert np.array_equal(kc2[rows[0]], r["k_int8"][0])


def _check_library_order(i):
    """The reference's own acceptance rule for this operator: int8 within 1 everywhere; scales and
    weights within 2.5e-5 absolute (query scale: up to 0.5 % of the entries may exceed it)."""
    r = lo.indexer_prolog_ref(*i.input_tensors())
    qi, qs, ki, ks, w = lo.indexer_prolog_library_order(*i.input_tensors()[:13])
    assert np.abs(r["q_int8"].astype(np.int32) - qi.numpy().astype(np.int32)).max() <= 1
    assert np.abs(r["k_int8"].astype(np.int32) - ki.numpy().astype(np.int32)).max() <= 1
    dq = np.abs(r["q_scale"].astype(np.float32) - qs.float().numpy())
    assert (dq > 2.5e-5).mean() <= 0.005
    assert np.abs(r["k_scale"].astype(np.float32) - ks.float().numpy()).max() <= 2.5e-5
    assert np.abs(r["weights"].astype(np.float32) - w.float().numpy()).max() <= 2.5e-5
    return r


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_small_case_against_library_order(seed):
    _check_library_order(_small(seed, affine_ln=(seed == 2)))


def test_reference_case_b4_s1_2_against_library_order():
    """Shapes of the reference's enabled test (b=4, s1=2, 64 K keys, h=7168, q_lora_rank=1536)."""
    i = gen_indexer_prolog_inputs(4, 2, [65536] * 4, seed=0)
    r = _check_library_order(i)
    assert r["q_int8"].shape == (8, 64, 128) and r["q_scale"].shape == (8, 64) and r["weights"].shape == (8, 64)
    assert np.isfinite(r["q_scale"].astype(np.float32)).all()
