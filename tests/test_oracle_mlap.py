"""Pins the MLA-prolog oracle (oracle/mlap_oracle.py).  The pieces it shares with the indexer-prolog oracle
(bf16 rounding, integer matmul, blocked sums over the hidden axis, int8 quantisation) are pinned in
tests/test_oracle_lip.py; here: the RMS norm and its sum order, the de-interleaving rope, the per-group
quantisation, the absorb product, the scatter, and the whole function against the golden evaluated with
torch's own matmul / sum at the reference's tolerances
(examples/models/deepseek_v32_exp/deepseekv32_mla_prolog_quant.py:668-692)."""
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import lip_oracle as lo
from oracle import mlap_oracle as mo
from pypto_amd.synthetic import gen_mla_prolog_inputs
from tests.test_oracle_lip import _bf16_int, _bf16_vals, _rn32


def test_rms_against_float64_and_order():
    rng = np.random.default_rng(0)
    v = _bf16_vals(rng, (5, 512), 7.0)
    gamma = _bf16_vals(rng, (512,), 1.0)
    got = mo.rms_fixed(v, gamma, 0.0).astype(np.float64)
    vd = v.astype(np.float64)
    exp = vd / np.sqrt((vd * vd).mean(-1, keepdims=True)) * gamma
    assert np.max(np.abs(got - exp)) <= 2.0 ** -8 * np.abs(exp).max()
    with_eps = mo.rms_fixed(v * np.float32(2.0 ** -12), gamma, 1e-5)             # epsilon matters for small rows
    assert np.abs(with_eps).max() < np.abs(mo.rms_fixed(v * np.float32(2.0 ** -12), gamma, 0.0)).max()
    # exact rational restatement of one row's sum order and arithmetic
    row = v[0]
    coef = float(np.float32(1.0 / 512))
    y = [_rn32(Fraction(_rn32(Fraction(float(a)) * Fraction(float(a)))) * Fraction(coef)) for a in row]
    s = 0.0
    for j in range(4):
        cur = y[128 * j:128 * j + 128]
        while len(cur) > 1:
            cur = [_rn32(Fraction(cur[i]) + Fraction(cur[i + 1])) for i in range(0, len(cur), 2)]
        s = _rn32(Fraction(s) + Fraction(cur[0]))
    d = float(np.sqrt(np.float32(s)))
    for c in (0, 130, 511):
        q = _rn32(Fraction(float(row[c])) / Fraction(d))
        want = _bf16_int(_rn32(Fraction(q) * Fraction(float(gamma[c]))))
        assert mo.rms_fixed(v[:1], gamma, 0.0)[0, c] == np.float32(want)


def test_rope_deinterleave_known_answer_and_rotation():
    v = np.arange(64, dtype=np.float32)[None, :]                                  # channel c holds c
    one, zero = np.ones((1, 64), np.float32), np.zeros((1, 64), np.float32)
    out = mo.rope_deinterleaved(v, one, zero)                                     # angle 0: only the permutation
    assert out[0, :32].tolist() == list(range(0, 64, 2)) and out[0, 32:].tolist() == list(range(1, 64, 2))
    out = mo.rope_deinterleaved(v, zero, one)                                     # angle pi/2: (a, b) -> (-b, a)
    assert out[0, :32].tolist() == [-float(c) for c in range(1, 64, 2)] and out[0, 32:].tolist() == list(range(0, 64, 2))
    rng = np.random.default_rng(1)
    x = _bf16_vals(rng, (3, 4, 64), 2.0)
    ang = rng.uniform(0, 2 * np.pi, (3, 64))
    cos, sin = lo.bf16_round(np.cos(ang).astype(np.float32)), lo.bf16_round(np.sin(ang).astype(np.float32))
    got = mo.rope_deinterleaved(x, cos, sin).astype(np.float64)
    a, b = x[..., 0::2].astype(np.float64), x[..., 1::2].astype(np.float64)
    c, s = cos.astype(np.float64)[:, None, :], sin.astype(np.float64)[:, None, :]
    exp = np.concatenate([a * c[..., :32] - b * s[..., :32], b * c[..., 32:] + a * s[..., 32:]], axis=-1)
    assert np.max(np.abs(got - exp)) <= 2.0 ** -8 * np.abs(exp).max()


def test_quant_rows_f32_known_answers():
    y = np.zeros((2, 4, 128), np.float32)
    y[0, 0, 3] = 2.0
    y[0, 0, 4] = -1.0
    y[0, 1, :] = np.linspace(-4, 4, 128, dtype=np.float32)
    q, s = mo.quant_rows_f32(lo.bf16_round(y))
    assert q[0, 0, 3] == 127 and q[0, 0, 4] == -64 and s[0, 0] == np.float32(1.0) / (np.float32(127.0) / np.float32(2.0))
    assert q[0, 1, 0] == -127 and q[0, 1, -1] == 127
    assert not q[0, 2].any() and s[0, 2] == 0 and s.dtype == np.float32             # all-zero group: zeros


def test_absorb_seq_rational_and_identity():
    rng = np.random.default_rng(2)
    a = _bf16_vals(rng, (2, 3, 128), 3.0)
    w = _bf16_vals(rng, (3, 128, 512), 0.1)
    got = mo.absorb_seq(a, w)
    for (t, n, c) in ((0, 0, 0), (1, 2, 511), (1, 1, 200)):
        acc = 0.0
        for i in range(128):
            acc = _rn32(Fraction(acc) + Fraction(float(a[t, n, i])) * Fraction(float(w[n, i, c])))
        assert got[t, n, c] == np.float32(_bf16_int(acc))
    eye = np.zeros((3, 128, 512), np.float32)
    eye[:, np.arange(128), np.arange(128)] = 1.0
    out = mo.absorb_seq(a, eye)
    assert np.array_equal(out[..., :128], a) and not out[..., 128:].any()


def _small(seed, **kw):
    args = dict(b=2, s1=2, act_seq=[300, 129], seed=seed, h=256, q_lora_rank=512, n_heads=4)
    args.update(kw)
    return gen_mla_prolog_inputs(**args)


def test_scatter_touches_only_named_rows():
    i = _small(3)
    r = mo.mla_prolog_ref(*i.input_tensors())
    rows = i.cache_index.numpy()
    for name, old, width in (("kv_cache", i.kv_cache.numpy(), 512), ("kr_cache", i.kr_cache.float().numpy(), 64),
                             ("k_scale_cache", i.k_scale_cache.numpy(), 4)):
        o, n = old.reshape(-1, width), r[name].reshape(-1, width)
        mask = np.ones(o.shape[0], bool)
        mask[rows] = False
        assert np.array_equal(o[mask], n[mask]), name
    assert np.array_equal(r["kv_cache"].reshape(-1, 512)[rows], r["k_int8"])
    assert np.array_equal(r["kr_cache"].reshape(-1, 64)[rows], r["k_rope"])
    assert np.array_equal(r["k_scale_cache"].reshape(-1, 4)[rows], r["k_scales"])


def _check_library_order(i):
    """The reference's own acceptance rule (deepseekv32_mla_prolog_quant.py:668-692): query parts atol 0.005 +
    rtol 2**-7 with up to 0.5 % outliers; int8 within 1; scales atol 2.5e-5 + rtol 0.005; rope atol 1e-4 + rtol 2**-7."""
    r = mo.mla_prolog_ref(*i.input_tensors())
    qn, qs, qnope, qrope, ki, kr, ks = mo.mla_prolog_library_order(*i.input_tensors()[:10])
    assert np.abs(r["q_norm"].astype(np.int32) - qn.numpy().astype(np.int32)).max() <= 1
    assert (np.abs(r["q_norm_scale"] - qs.numpy()) <= 2.5e-5 + 0.005 * np.abs(qs.numpy())).all()
    for g, ref in ((r["query_nope"], qnope.float().numpy()), (r["query_rope"], qrope.float().numpy())):
        assert (np.abs(g - ref) > 0.005 + 0.0078125 * np.abs(ref)).mean() <= 0.005
    assert np.abs(r["k_int8"].astype(np.int32) - ki.numpy().astype(np.int32)).max() <= 1
    assert (np.abs(r["k_rope"] - kr.float().numpy()) <= 1e-4 + 0.0078125 * np.abs(kr.float().numpy())).all()
    assert (np.abs(r["k_scales"] - ks.numpy()) <= 2.5e-5 + 0.005 * np.abs(ks.numpy())).all()
    return r


@pytest.mark.parametrize("seed", [0, 1])
def test_small_case_against_library_order(seed):
    _check_library_order(_small(seed))


def test_reference_case_b4_s2_against_library_order():
    """Shapes of the reference's enabled test (b=4, s=2, 128 heads, h=7168, q_lora_rank=1536, 4 K keys)."""
    r = _check_library_order(gen_mla_prolog_inputs(4, 2, [4096] * 4, seed=0))
    assert r["query_nope"].shape == (8, 128, 512) and r["query_rope"].shape == (8, 128, 64) and r["q_norm"].shape == (8, 1536)
