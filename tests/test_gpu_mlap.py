"""Parity of the HIP MLA prolog (through the operator, pybind11 and the C ABI) against the CPU oracle.  The
oracle fixes the order of every fp32 sum, so the bar is bit-exact for every output: int8 query latent and
its fp32 scale, bf16 absorbed query (nope and rope parts), and every byte of the three caches."""
import numpy as np
import pytest
import torch

import pypto_amd
from oracle import mlap_oracle as mo
from pypto_amd.synthetic import gen_mla_prolog_inputs
from pypto_amd.utils.compare import compare

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def exact_absorb():
    """The bit-exact tests run both prologs with every sum in its fixed order; the matrix-core forms have tests of
    their own that switch them on."""
    from pypto_amd import lightning_indexer_prolog_quant_impl as lip_impl
    from pypto_amd import mla_prolog_quant_impl as impl
    old = impl.EXACT_ABSORB, lip_impl.EXACT_SUMS, lip_impl.MATRIX_CORE_HIDDEN_SUMS
    impl.EXACT_ABSORB = True
    lip_impl.EXACT_SUMS = True
    yield
    impl.EXACT_ABSORB, lip_impl.EXACT_SUMS, lip_impl.MATRIX_CORE_HIDDEN_SUMS = old


def run_op(inp, eps=(0.0, 0.0), separate_cache_out=False, prefill=False, cache_mode="PA_BSND"):
    dev = torch.device("cuda:0")
    d = inp.to(dev)
    t, n, ql = d.token_x.shape[0], d.w_uk.shape[0], d.w_dq.shape[1]
    q_norm = torch.full([t, ql], -7, dtype=torch.int8, device=dev)
    q_norm_scale = torch.full([t, 1], -7.0, dtype=torch.float32, device=dev)
    q_nope = torch.full([t, n, 512], -7.0, dtype=torch.bfloat16, device=dev)
    q_rope = torch.full([t, n, 64], -7.0, dtype=torch.bfloat16, device=dev)
    if separate_cache_out:
        kv, kr, ks = torch.zeros_like(d.kv_cache), torch.zeros_like(d.kr_cache), torch.zeros_like(d.k_scale_cache)
    else:
        kv, kr, ks = d.kv_cache, d.kr_cache, d.k_scale_cache
    ins = [pypto_amd.from_torch(v) for v in d.input_tensors()]
    outs = [pypto_amd.from_torch(v) for v in (q_norm, q_norm_scale, q_nope, q_rope, kv, kr, ks)]
    fn = pypto_amd.mla_prolog_quant_p if prefill else pypto_amd.mla_prolog_quant_d
    ret = fn(*ins, *outs, eps[0], eps[1], cache_mode, pypto_amd.MlaTileConfig(), pypto_amd.RopeTileShapeConfig())
    assert ret is None
    torch.cuda.synchronize()
    return {"q_norm": q_norm.cpu().numpy(), "q_norm_scale": q_norm_scale.cpu().numpy()[:, 0],
            "query_nope": q_nope.float().cpu().numpy(), "query_rope": q_rope.float().cpu().numpy(),
            "kv_cache": kv.cpu().numpy(), "kr_cache": kr.float().cpu().numpy(), "k_scale_cache": ks.cpu().numpy()}


# The reference driver's acceptance rule for the quantised variant, output by output: (atol, rtol, share of elements
# that may lie outside atol + rtol * |ref|), deepseekv32_mla_prolog_quant.py:672-692.  The bound is per element and
# the three caches allow no outlier at all.
REFERENCE_RULE = {
    "query_nope": (0.005, 0.0078125, 0.005), "query_rope": (0.005, 0.0078125, 0.005),
    "q_norm": (1.0, 0.0, 0.005), "q_norm_scale": (0.000025, 0.005, 0.005),
    "kv_cache": (1.0, 0.0, 0), "kr_cache": (0.0001, 0.0078125, 0), "k_scale_cache": (0.000025, 0.005, 0),
}


def assert_reference_rule(got, ref, rows, what):
    """compare() of the reference with its own triples; cache outputs are looked at in the rows the call wrote."""
    for name, (atol, rtol, ratio) in REFERENCE_RULE.items():
        g, r = np.asarray(got[name]), np.asarray(ref[name])
        if name.endswith("_cache"):
            g = g.reshape(-1, g.shape[-1])[rows]
            if r.ndim != 2 or r.shape[0] != len(rows):
                r = r.reshape(-1, r.shape[-1])[rows]
        r = r.reshape(g.shape)
        compare(torch.from_numpy(np.ascontiguousarray(g)), torch.from_numpy(np.ascontiguousarray(r)), f"{what}: {name}", atol, rtol, ratio)


def assert_exact(got, ref, what):
    for name in ("q_norm", "q_norm_scale", "query_nope", "query_rope", "kv_cache", "kr_cache", "k_scale_cache"):
        g, r = got[name], ref[name]
        assert g.shape == r.shape, (what, name, g.shape, r.shape)
        gi = g.view(np.uint8) if g.dtype == np.int8 else g.view(np.uint32)
        ri = r.view(np.uint8) if r.dtype == np.int8 else r.view(np.uint32)
        if not np.array_equal(gi, ri):
            bad = np.argwhere(gi != ri)
            first = tuple(bad[0])
            raise AssertionError(f"{what}: {name}: {len(bad)} of {g.size} differ; first at {first}: got {g[first]} want {r[first]}")


@pytest.mark.parametrize("b,s1,act,kw,eps", [
    (2, 2, [300, 129], dict(h=256, q_lora_rank=512, n_heads=4), (0.0, 0.0)),        # small everything, golden's norm
    (1, 1, [77], dict(h=1152, q_lora_rank=1024, n_heads=2), (1e-5, 1e-5)),          # one token, ragged last group (18 blocks)
    (3, 1, [5, 128, 129], dict(h=512, q_lora_rank=1536, n_heads=8), (1e-5, 1e-6)),
    (5, 7, [900] * 5, dict(h=192, q_lora_rank=512, n_heads=2), (1e-5, 1e-5)),       # 35 tokens: ragged groups of 8, two token blocks
])
def test_mla_prolog_small_shapes_bit_exact(b, s1, act, kw, eps):
    inp = gen_mla_prolog_inputs(b, s1, act, seed=3 * b + s1, **kw)
    ref = mo.mla_prolog_ref(*inp.input_tensors(), epsilon_cq=eps[0], epsilon_ckv=eps[1])
    assert_exact(run_op(inp, eps), ref, f"b={b} s1={s1} {kw}")


def test_mla_prolog_cache_mode_pa_nz_is_accepted_and_changes_nothing():
    """The reference asserts cache_mode in ("PA_BSND", "PA_NZ") and does nothing else with it
    (mla_prolog_quant_impl.py:591): both values give the same outputs and cache rows."""
    inp = gen_mla_prolog_inputs(2, 2, [300, 129], seed=8, h=256, q_lora_rank=512, n_heads=4)
    ref = mo.mla_prolog_ref(*inp.input_tensors(), epsilon_cq=1e-5, epsilon_ckv=1e-5)
    assert_exact(run_op(inp, (1e-5, 1e-5), cache_mode="PA_NZ"), ref, "PA_NZ")


def test_mla_prolog_reference_case_b4_s2():
    """Shapes of the reference's enabled test (deepseekv32_mla_prolog_quant.py:790-834): b=4, s=2, 128 heads,
    h=7168, q_lora_rank=1536, epsilons 1e-5 as its driver passes them."""
    inp = gen_mla_prolog_inputs(4, 2, [4096] * 4, seed=0)
    ref = mo.mla_prolog_ref(*inp.input_tensors(), epsilon_cq=1e-5, epsilon_ckv=1e-5)
    got = run_op(inp, (1e-5, 1e-5))
    assert_exact(got, ref, "b4_s2")
    # and the reference's own acceptance rule against the library-order evaluation of its golden
    qn, qs, qnope, qrope, ki, kr, ks = mo.mla_prolog_library_order(*inp.input_tensors()[:10])
    rows = inp.cache_index.numpy()
    lib = {"q_norm": qn.numpy(), "q_norm_scale": qs.numpy().reshape(-1), "query_nope": qnope.float().numpy(),
           "query_rope": qrope.float().numpy(), "kv_cache": ki.numpy(), "kr_cache": kr.float().numpy(), "k_scale_cache": ks.numpy()}
    assert_reference_rule(got, lib, rows, "b4_s2 against the library-order golden")


def test_mla_prolog_matrix_core_absorb_default():
    """The operator's default: query_nope summed on the matrix cores.  Everything but query_nope stays bit-exact;
    query_nope meets the reference's acceptance rule for it (deepseekv32_mla_prolog_quant.py:668-692: at most
    0.5 % of the elements off by more than 0.005 + 2^-7 |ref|) against the sequential statement, and in fact
    differs from it by at most one bf16 step."""
    from pypto_amd import mla_prolog_quant_impl as impl
    impl.EXACT_ABSORB = False
    for b, s1, act, kw in ((4, 2, [4096] * 4, {}), (2, 3, [900] * 2, dict(h=192, q_lora_rank=512, n_heads=2))):   # 8 and 6 tokens
        inp = gen_mla_prolog_inputs(b, s1, act, seed=31 + b, **kw)
        ref = mo.mla_prolog_ref(*inp.input_tensors(), epsilon_cq=1e-5, epsilon_ckv=1e-5)
        got = run_op(inp, (1e-5, 1e-5))
        for name in ("q_norm", "q_norm_scale", "query_rope", "kv_cache", "kr_cache", "k_scale_cache"):
            g, r = got[name], ref[name]
            assert np.array_equal(g.view(np.uint8) if g.dtype == np.int8 else g.view(np.uint32),
                                  r.view(np.uint8) if r.dtype == np.int8 else r.view(np.uint32)), name
        assert_reference_rule(got, ref, inp.cache_index.numpy(), f"b={b} s1={s1}, matrix-core absorb")
        g, r = got["query_nope"], ref["query_nope"]
        assert np.abs(g - r).max() <= 0.0079 * np.abs(r).max()
        print(f"b={b} s1={s1}: query_nope elements that differ from the sequential sums: {float((g != r).mean()):.4f}", flush=True)


def test_mla_prolog_prefill_t512():
    """mla_prolog_quant_p on one sequence of 512 tokens at full size, the largest case the reference carries for
    this operator (deepseekv32_mla_indexer_prolog_quant.py:1049-1050, t_512): bit-exact like the decode cases."""
    inp = gen_mla_prolog_inputs(1, 512, [4096], seed=21)
    ref = mo.mla_prolog_ref(*inp.input_tensors(), epsilon_cq=1e-5, epsilon_ckv=1e-5)
    assert_exact(run_op(inp, (1e-5, 1e-5), prefill=True), ref, "t_512 prefill")


def test_mla_prolog_prefill_t512_matrix_core_sums_default():
    """The operator's default from 9 tokens on: the sums over the hidden axis run on the matrix cores as well
    (same exact products, the cores' own summation order; the 64 rope columns excepted, which stay in the fixed order),
    so the int8 latents may differ by one step where the sequential sums land next to a rounding boundary.  Held to the reference's acceptance rule for every output
    (deepseekv32_mla_prolog_quant.py:668-692) against the sequential statement; a short-h shape with ragged
    token tiles and a half-empty chunk split rides along, and the decode batches that take these forms: 16 and 32
    tokens at the model's sizes, 9, 39 and 63 (ragged blocks of 32) at small ones."""
    from pypto_amd import mla_prolog_quant_impl as impl
    impl.EXACT_ABSORB = False
    small = dict(h=192, q_lora_rank=512, n_heads=2)
    for b, s1, act, kw in ((1, 512, [4096], {}), (3, 50, [700] * 3, small), (16, 1, [4096] * 16, {}), (32, 1, [4096] * 32, {}),
                           (3, 13, [700] * 3, small), (9, 7, [300] * 9, small), (9, 1, [300] * 9, small)):
        inp = gen_mla_prolog_inputs(b, s1, act, seed=41 + b, **kw)
        ref = mo.mla_prolog_ref(*inp.input_tensors(), epsilon_cq=1e-5, epsilon_ckv=1e-5)
        got = run_op(inp, (1e-5, 1e-5), prefill=True)
        rows = inp.cache_index.numpy()
        assert_reference_rule(got, ref, rows, f"t={b * s1}, matrix-core sums")
        # the rotated key keeps its fixed-order sums in every mode (the rule allows it no outlier): the same bits
        assert np.array_equal(got["kr_cache"].reshape(-1, 64)[rows].view(np.uint32), ref["kr_cache"].reshape(-1, 64)[rows].view(np.uint32))
        dq = np.abs(got["q_norm"].astype(np.int32) - ref["q_norm"].astype(np.int32))
        assert dq.max() <= 1 and (dq != 0).mean() <= 0.01
        gk, rk = got["kv_cache"].reshape(-1, 512)[rows].astype(np.int32), ref["kv_cache"].reshape(-1, 512)[rows].astype(np.int32)
        assert np.abs(gk - rk).max() <= 1 and (gk != rk).mean() <= 0.01
        print(f"t={b * s1}: q_norm entries off by one {float((dq != 0).mean()):.5f}, latent entries off by one {float((gk != rk).mean()):.5f}", flush=True)


def test_mla_prolog_separate_cache_output_skipped_indices_and_repeatability():
    inp = gen_mla_prolog_inputs(2, 2, [300, 129], seed=5, h=256, q_lora_rank=512, n_heads=4)
    inp.cache_index[1] = -1
    inp.cache_index[2] = inp.kv_cache.shape[0] * inp.kv_cache.shape[1]
    ref = mo.mla_prolog_ref(*inp.input_tensors(), epsilon_cq=1e-5, epsilon_ckv=1e-5)
    a = run_op(inp, (1e-5, 1e-5), separate_cache_out=True, prefill=True)
    assert_exact(a, ref, "separate outputs, two skipped indices")
    assert_exact(run_op(inp, (1e-5, 1e-5), separate_cache_out=True), a, "second run")


def test_mla_prolog_feeds_the_attention_cache_layout():
    """The rows the prolog writes are the rows the attention reads: int8 latent, four fp32 scales, bf16 rope,
    at the page-table position of the newest tokens.  De-quantising them reproduces the normalised latent."""
    inp = gen_mla_prolog_inputs(2, 1, [200, 131], seed=8, h=256, q_lora_rank=512, n_heads=2)
    got = run_op(inp, (1e-5, 1e-5))
    ref = mo.mla_prolog_ref(*inp.input_tensors(), epsilon_cq=1e-5, epsilon_ckv=1e-5)
    table = inp.block_table.numpy()
    for bi, a in enumerate(inp.act_seq):
        row = table[bi, (a - 1) // 128] * 128 + (a - 1) % 128
        assert row == int(inp.cache_index[bi])
        deq = got["kv_cache"].reshape(-1, 512)[row].astype(np.float32).reshape(4, 128) * got["k_scale_cache"].reshape(-1, 4)[row][:, None]
        np.testing.assert_array_equal(got["kv_cache"].reshape(-1, 512)[row], ref["k_int8"][bi])
        assert np.abs(deq.reshape(512)).max() > 0


def run_fused(dm, dl, t, n, n_idx, op=None):
    """The fused operator on device inputs dm (MLA prolog) and dl (indexer prolog); caches updated in place."""
    dev = dm.token_x.device
    q_nope = torch.empty([t, n, 512], dtype=torch.bfloat16, device=dev)
    q_rope = torch.empty([t, n, 64], dtype=torch.bfloat16, device=dev)
    q_int8 = torch.empty([t, n_idx, 128], dtype=torch.int8, device=dev)
    q_scale = torch.empty([t, n_idx, 1], dtype=torch.float16, device=dev)
    weights = torch.empty([t, n_idx], dtype=torch.float16, device=dev)
    ret = (op or pypto_amd.mla_indexer_prolog_quant_d)(
        dm.token_x, dm.w_dq, dm.w_uq_qr, dm.dequant_scale, dm.w_uk, dm.w_dkv_kr, dm.gamma_cq, dm.gamma_ckv, dm.cos, dm.sin,
        dm.cache_index, dm.kv_cache, dm.kr_cache, dm.k_scale_cache, dl.w_qb, dl.w_qb_scale, dl.wk, dl.w_proj, dl.ln_gamma_k,
        dl.ln_beta_k, dl.hadamard_q, dl.hadamard_k, dl.k_cache, dl.k_cache_scale, q_nope, q_rope, dm.kv_cache, dm.kr_cache,
        dm.k_scale_cache, q_int8, q_scale, dl.k_cache, dl.k_cache_scale, weights, 1e-5, 1e-5, "PA_BSND",
        pypto_amd.MlaTileConfig(), pypto_amd.IndexerPrologQuantAttr(), pypto_amd.IndexerPrologQuantConfigs(),
        pypto_amd.RopeTileShapeConfig())
    assert ret is None
    torch.cuda.synchronize()
    return q_nope, q_rope, q_int8, q_scale, weights


@pytest.mark.parametrize("mode,shape", [("default", "small"), ("exact", "small"), ("matrix_cores", "small"), ("default", "t_512"),
                                        ("default", "t_11_idx_64"), ("exact", "t_11_idx_64"), ("default", "t_3_idx_32"),
                                        ("default", "t_40_idx_64"), ("exact", "t_40_idx_64"), ("default", "t_7_idx_64"),
                                        ("default", "t_32_idx_64")])
def test_fused_prolog_at_prefill_size_equals_the_two_operators_chained(mode, shape):
    """150 tokens (ragged last block of the token tiles): the fused operator's prefill-sized launches (unsplit int8
    projections, the attention query's last stage per head and run of token blocks) against the MLA prolog and the
    indexer prolog called one after the other on the same inputs, bit for bit, in each of the summation modes.
    The two decode-sized shapes: with 64 indexer heads the indexer prolog's first stage rides in the MLA prolog's
    launches (7 tokens by default; 11 in the exact mode: two token groups, the second ragged; 576 hidden channels: a
    second, short group of blocks), with 32 heads it keeps its own launch.  At 40 tokens the MLA half takes its prefill forms by default
    while the indexer half keeps its decode forms (in the exact mode both keep them, and the rider); at 32 and at 11
    tokens the two last stages share a launch as well."""
    from pypto_amd import lightning_indexer_prolog_quant_impl as lip_impl
    from pypto_amd import mla_prolog_quant_impl as impl
    from pypto_amd.synthetic import gen_indexer_prolog_inputs
    impl.EXACT_ABSORB = lip_impl.EXACT_SUMS = mode == "exact"
    lip_impl.MATRIX_CORE_HIDDEN_SUMS = mode == "matrix_cores"
    if shape == "small":
        kw = dict(h=256, q_lora_rank=512)
        b, s1, act, n_mla, n_idx = 3, 50, [700, 650, 600], 4, 8
    elif shape == "t_11_idx_64":
        kw = dict(h=576, q_lora_rank=512)
        b, s1, act, n_mla, n_idx = 11, 1, [700 - 37 * i for i in range(11)], 4, 64
    elif shape == "t_7_idx_64":
        kw = dict(h=576, q_lora_rank=512)
        b, s1, act, n_mla, n_idx = 7, 1, [700 - 37 * i for i in range(7)], 4, 64
    elif shape == "t_40_idx_64":
        kw = dict(h=576, q_lora_rank=512)
        b, s1, act, n_mla, n_idx = 5, 8, [700, 650, 600, 550, 500], 4, 64
    elif shape == "t_32_idx_64":
        kw = dict(h=576, q_lora_rank=512)
        b, s1, act, n_mla, n_idx = 4, 8, [700, 650, 600, 550], 4, 64
    elif shape == "t_3_idx_32":
        kw = dict(h=576, q_lora_rank=512)
        b, s1, act, n_mla, n_idx = 3, 1, [700, 650, 600], 4, 32
    else:   # the reference's test_t_512_tilebs_128_p (deepseekv32_mla_indexer_prolog_quant.py:1050-1117) at the model's sizes
        kw = {}
        b, s1, act, n_mla, n_idx = 128, 4, [4096] * 128, 128, 64
    dev = torch.device("cuda:0")
    mla = gen_mla_prolog_inputs(b, s1, act, seed=31, n_heads=n_mla, **kw)
    lip = gen_indexer_prolog_inputs(b, s1, act, seed=32, n_heads=n_idx, **kw)
    t = b * s1
    # separate operators
    sep = run_op(mla, (1e-5, 1e-5), prefill=True)
    dl = lip.to(dev)
    la = list(dl.input_tensors())
    dm0 = mla.to(dev)
    la[0], la[1], la[2] = dm0.token_x, torch.from_numpy(sep["q_norm"]).to(dev), torch.from_numpy(sep["q_norm_scale"]).reshape(-1, 1).to(dev)
    la[9], la[10], la[15] = dm0.cos, dm0.sin, dm0.cache_index
    s_q = torch.empty([t, n_idx, 128], dtype=torch.int8, device=dev)
    s_sc = torch.empty([t, n_idx, 1], dtype=torch.float16, device=dev)
    s_w = torch.empty([t, n_idx], dtype=torch.float16, device=dev)
    pypto_amd.lightning_indexer_prolog_quant(*la, s_q, s_sc, dl.k_cache, dl.k_cache_scale, s_w)
    torch.cuda.synchronize()
    # fused
    dm, dl2 = mla.to(dev), lip.to(dev)
    q_nope, q_rope, q_int8, q_scale, weights = run_fused(dm, dl2, t, n_mla, n_idx, op=pypto_amd.mla_indexer_prolog_quant_p)
    assert np.array_equal(q_nope.float().cpu().numpy(), sep["query_nope"])
    assert np.array_equal(q_rope.float().cpu().numpy(), sep["query_rope"])
    assert np.array_equal(dm.kv_cache.cpu().numpy(), sep["kv_cache"])
    assert np.array_equal(dm.kr_cache.float().cpu().numpy(), sep["kr_cache"])
    assert torch.equal(q_int8, s_q) and torch.equal(q_scale, s_sc) and torch.equal(weights, s_w)
    assert torch.equal(dl2.k_cache, dl.k_cache) and torch.equal(dl2.k_cache_scale, dl.k_cache_scale)


def test_fused_mla_indexer_prolog_matches_the_oracle_chain():
    """mla_indexer_prolog_quant_d: the indexer prolog consumes the MLA prolog's hidden q_norm / q_norm_scale; the
    ten outputs equal the two oracles chained (cos/sin of the MLA generator's range feed both stages)."""
    from oracle import lip_oracle as lo
    from pypto_amd.synthetic import gen_indexer_prolog_inputs
    kw = dict(h=256, q_lora_rank=512)
    mla = gen_mla_prolog_inputs(2, 2, [300, 129], seed=14, n_heads=4, **kw)
    lip = gen_indexer_prolog_inputs(2, 2, [300, 129], seed=15, n_heads=4, **kw)
    assert lip.k_cache.shape[0] == mla.kv_cache.shape[0]
    r_mla = mo.mla_prolog_ref(*mla.input_tensors(), epsilon_cq=1e-5, epsilon_ckv=1e-5)
    la = list(lip.input_tensors())
    la[0], la[1], la[2] = mla.token_x, torch.from_numpy(r_mla["q_norm"]), torch.from_numpy(r_mla["q_norm_scale"]).reshape(-1, 1)
    la[9], la[10], la[15] = mla.cos, mla.sin, mla.cache_index
    r_lip = lo.indexer_prolog_ref(*la)

    dev = torch.device("cuda:0")
    dm, dl = mla.to(dev), lip.to(dev)
    q_nope, q_rope, q_int8, q_scale, weights = run_fused(dm, dl, 4, 4, 4)
    assert np.array_equal(q_nope.float().cpu().numpy(), r_mla["query_nope"])
    assert np.array_equal(q_rope.float().cpu().numpy(), r_mla["query_rope"])
    assert np.array_equal(dm.kv_cache.cpu().numpy(), r_mla["kv_cache"])
    assert np.array_equal(q_int8.cpu().numpy(), r_lip["q_int8"])
    assert np.array_equal(q_scale.cpu().numpy()[..., 0].view(np.uint16), r_lip["q_scale"].view(np.uint16))
    assert np.array_equal(weights.cpu().numpy().view(np.uint16), r_lip["weights"].view(np.uint16))
    assert np.array_equal(dl.k_cache.cpu().numpy(), r_lip["k_cache"])
    assert np.array_equal(dl.k_cache_scale.cpu().numpy().view(np.uint16), r_lip["k_cache_scale"].view(np.uint16))


def test_fused_entry_point_through_the_c_abi_keeps_the_intermediates_in_its_workspace():
    """pto_mla_indexer_prolog_quant_launch called with ctypes, q_norm_out / q_norm_scale_out NULL: the query latent
    lives in the common workspace, and every output equals what the two operators give when called one after
    the other (bit for bit)."""
    import ctypes
    import os
    from pypto_amd.synthetic import gen_indexer_prolog_inputs
    lib = ctypes.CDLL(os.path.join(os.path.dirname(os.path.abspath(pypto_amd.__file__)), "libpypto_amd_sfa.so"))
    vp, i64, f32, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_float, ctypes.c_int32

    class Mla(ctypes.Structure):
        _fields_ = [(n, vp) for n in ("token_x", "w_dq", "w_uq_qr", "dequant_scale", "w_uk", "w_dkv_kr", "gamma_cq", "gamma_ckv",
                                      "cos", "sin", "cache_index", "kv_cache", "kr_cache", "k_scale_cache", "q_norm_out",
                                      "q_norm_scale_out", "query_nope_out", "query_rope_out", "workspace")] + \
                   [("workspace_bytes", ctypes.c_size_t)] + [(n, i64) for n in ("t", "h", "q_lora_rank", "n_heads", "cache_rows")] + \
                   [("epsilon_cq", f32), ("epsilon_ckv", f32), ("absorb_exact", i32), ("reserved", i32)]

    class Idx(ctypes.Structure):
        _fields_ = [(n, vp) for n in ("x", "q_norm", "q_norm_scale", "w_qb", "w_qb_scale", "wk", "w_proj", "ln_gamma_k", "ln_beta_k",
                                      "cos_idx_rope", "sin_idx_rope", "hadamard_q", "hadamard_k", "k_cache", "k_cache_scale",
                                      "k_cache_index", "q_int8", "q_scale", "weights", "workspace")] + \
                   [("workspace_bytes", ctypes.c_size_t)] + [(n, i64) for n in ("t", "h", "q_lora_rank", "n_heads", "cache_rows")] + \
                   [("eps", f32), ("sum_mode", i32)]

    class Fused(ctypes.Structure):
        _fields_ = [("mla", Mla), ("indexer", Idx), ("workspace", vp), ("workspace_bytes", ctypes.c_size_t)]

    kw = dict(h=512, q_lora_rank=512)
    mla = gen_mla_prolog_inputs(3, 2, [300, 129, 64], seed=31, n_heads=8, **kw)
    lip = gen_indexer_prolog_inputs(3, 2, [300, 129, 64], seed=32, n_heads=8, **kw)
    dev = torch.device("cuda:0")
    t, n = 6, 8

    def outputs():
        dm, dl = mla.to(dev), lip.to(dev)
        return dm, dl, dict(q_nope=torch.zeros([t, n, 512], dtype=torch.bfloat16, device=dev),
                            q_rope=torch.zeros([t, n, 64], dtype=torch.bfloat16, device=dev),
                            q_int8=torch.zeros([t, n, 128], dtype=torch.int8, device=dev),
                            q_scale=torch.zeros([t, n, 1], dtype=torch.float16, device=dev),
                            weights=torch.zeros([t, n], dtype=torch.float16, device=dev))

    # the two operators one after the other
    dm, dl, o = outputs()
    q_norm = torch.zeros([t, 512], dtype=torch.int8, device=dev)
    q_norm_scale = torch.zeros([t, 1], dtype=torch.float32, device=dev)
    pypto_amd.mla_prolog_quant_d(dm.token_x, dm.w_dq, dm.w_uq_qr, dm.dequant_scale, dm.w_uk, dm.w_dkv_kr, dm.gamma_cq, dm.gamma_ckv,
                                 dm.cos, dm.sin, dm.cache_index, dm.kv_cache, dm.kr_cache, dm.k_scale_cache, q_norm, q_norm_scale,
                                 o["q_nope"], o["q_rope"], dm.kv_cache, dm.kr_cache, dm.k_scale_cache, 1e-5, 1e-5)
    pypto_amd.lightning_indexer_prolog_quant(dm.token_x, q_norm, q_norm_scale, dl.w_qb, dl.w_qb_scale, dl.wk, dl.w_proj, dl.ln_gamma_k,
                                             dl.ln_beta_k, dm.cos, dm.sin, dl.hadamard_q, dl.hadamard_k, dl.k_cache, dl.k_cache_scale,
                                             dm.cache_index, o["q_int8"], o["q_scale"], dl.k_cache, dl.k_cache_scale, o["weights"])
    torch.cuda.synchronize()
    want = {k: v.clone() for k, v in o.items()}
    want.update(kv=dm.kv_cache.clone(), kr=dm.kr_cache.clone(), ks=dm.k_scale_cache.clone(), kc=dl.k_cache.clone(), kcs=dl.k_cache_scale.clone())

    # the fused entry point
    dm, dl, o = outputs()
    a = Fused()
    for name, ten in (("token_x", dm.token_x), ("w_dq", dm.w_dq), ("w_uq_qr", dm.w_uq_qr), ("dequant_scale", dm.dequant_scale),
                      ("w_uk", dm.w_uk), ("w_dkv_kr", dm.w_dkv_kr), ("gamma_cq", dm.gamma_cq), ("gamma_ckv", dm.gamma_ckv),
                      ("cos", dm.cos), ("sin", dm.sin), ("cache_index", dm.cache_index), ("kv_cache", dm.kv_cache),
                      ("kr_cache", dm.kr_cache), ("k_scale_cache", dm.k_scale_cache), ("query_nope_out", o["q_nope"]),
                      ("query_rope_out", o["q_rope"])):
        setattr(a.mla, name, ten.data_ptr())
    a.mla.t, a.mla.h, a.mla.q_lora_rank, a.mla.n_heads = t, 512, 512, n
    a.mla.cache_rows = dm.kv_cache.shape[0] * dm.kv_cache.shape[1]
    a.mla.epsilon_cq = a.mla.epsilon_ckv = 1e-5
    a.mla.absorb_exact = 1                                   # the autouse fixture runs the separate operators that way
    for name, ten in (("w_qb", dl.w_qb), ("w_qb_scale", dl.w_qb_scale), ("wk", dl.wk), ("w_proj", dl.w_proj),
                      ("ln_gamma_k", dl.ln_gamma_k), ("ln_beta_k", dl.ln_beta_k), ("hadamard_q", dl.hadamard_q),
                      ("hadamard_k", dl.hadamard_k), ("k_cache", dl.k_cache), ("k_cache_scale", dl.k_cache_scale),
                      ("q_int8", o["q_int8"]), ("q_scale", o["q_scale"]), ("weights", o["weights"])):
        setattr(a.indexer, name, ten.data_ptr())
    a.indexer.n_heads = n
    a.indexer.cache_rows = dl.k_cache.shape[0] * dl.k_cache.shape[1]
    a.indexer.eps = 1e-6
    need = ctypes.c_size_t()
    assert lib.pto_mla_indexer_prolog_quant_workspace_bytes(ctypes.byref(a), ctypes.byref(need)) == 0
    ws = torch.empty(need.value, dtype=torch.uint8, device=dev)
    a.workspace, a.workspace_bytes = ws.data_ptr(), need.value
    lib.pto_last_error.restype = ctypes.c_char_p
    rc = lib.pto_mla_indexer_prolog_quant_launch(ctypes.byref(a), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, lib.pto_last_error()
    torch.cuda.synchronize()
    got = dict(o, kv=dm.kv_cache, kr=dm.kr_cache, ks=dm.k_scale_cache, kc=dl.k_cache, kcs=dl.k_cache_scale)
    for k in want:
        assert torch.equal(got[k].view(torch.uint8), want[k].view(torch.uint8)), k
    # the intermediates sit at the front of the workspace
    assert torch.equal(ws[:t * 512].view(torch.int8).view(t, 512), q_norm)
    # a workspace one byte short is refused, nothing is launched
    a.workspace_bytes = need.value - 1
    assert lib.pto_mla_indexer_prolog_quant_launch(ctypes.byref(a), None) == -2
