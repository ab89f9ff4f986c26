"""The benchmark configurations at their full sizes on the GPU: the chained path of configuration 2
(indexer -> attention), configuration 3 (two query tokens per sequence) and configuration 4 (a 4096-token
prefill), against the C statement of the goldens and through properties that hold at any size."""
import pytest
import torch

import pypto_amd
from pypto_amd.synthetic import config_lengths, gen_indexer_inputs, gen_sfa_inputs
from pypto_amd.utils import attention_error_stats

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_REL = 2e-2, 5e-3
DEV = "cuda:0"


def run_sfa(inp, topk_indices=None):
    d = inp.to(torch.device(DEV))
    out = torch.full([inp.b, inp.s1, inp.n_q, 512], float("nan"), dtype=torch.bfloat16, device=DEV)
    ti = d.topk_indices if topk_indices is None else topk_indices
    pypto_amd.sparse_flash_attention_quant_d(d.query_nope, d.query_rope, d.key_nope_2d, d.key_rope_2d,
                                             d.k_nope_scales, ti, d.block_table, d.kv_act_seqs, out, inp.n_q, 1,
                                             inp.softmax_scale, inp.topk, inp.block_size, inp.max_blocknum_perbatch,
                                             None)
    torch.cuda.synchronize()
    return out.cpu()


def golden(c_oracle, inp, topk_indices=None):
    ti = inp.topk_indices if topk_indices is None else topk_indices
    return c_oracle.sfa_quant(inp.query_nope, inp.query_rope, inp.key_nope_2d, inp.key_rope_2d, inp.k_nope_scales, ti,
                              inp.block_table, inp.kv_act_seqs, inp.b, inp.s1, inp.n_q, inp.topk, inp.block_size,
                              inp.softmax_scale, s2_tile=0)


def check(out, ref, what):
    assert not torch.isnan(out).any(), f"{what}: NaN in output"
    max_abs, mean_rel = attention_error_stats(out, ref)
    print(f"{what}: max_abs={max_abs:.4g} mean_rel={mean_rel:.4g}", flush=True)
    assert max_abs <= MAX_ABS and mean_rel <= MEAN_REL, (what, max_abs, mean_rel)


def assert_close_to_fp64_truth(out, gold, inp, rows, what, topk_indices=None):
    """The sharper bar at full size.  At top-k 2048 an output element is a softmax-weighted mean of 2048 values and
    about 0.03 in magnitude, so the max-abs bound of 2e-2 says little there.  For a sample of query rows (b, s1)
    the exact attention -- fp64 scores, softmax and weighted sum over the same de-quantised bf16 keys the golden
    uses -- is formed, and the kernel's mean-rel error against it may exceed the single-pass golden's own error
    (its bf16 probabilities and bf16 result) by a quarter at most."""
    from oracle import sfa_oracle as so
    ti = inp.topk_indices if topk_indices is None else topk_indices
    ti = ti.reshape(inp.b * inp.s1, -1).long()
    num_k = den = num_g = 0.0
    for b, s1 in rows:
        cur = min(max(int(inp.actual_seq[b]) - inp.s1 + 1 + s1, 0), inp.topk)
        assert cur > 0, "sample rows must see keys"
        idx = ti[b * inp.s1 + s1, :cur]
        phys = inp.block_table[b].long()[idx // inp.block_size] * inp.block_size + idx % inp.block_size
        kn = so.dequant_kn(inp.key_nope_2d[phys], inp.k_nope_scales[phys]).double()
        k = torch.cat([kn, inp.key_rope_2d[phys].double()], dim=-1)
        q = inp.q_bsnd()[b, s1].double()                                    # [heads, 576]
        p = torch.softmax((q @ k.T) * inp.softmax_scale, dim=-1)
        truth = p @ kn                                                      # [heads, 512]
        num_k += float((out[b, s1].double() - truth).abs().sum())
        num_g += float((gold[b, s1].double() - truth).abs().sum())
        den += float(truth.abs().sum())
    err_k, err_g = num_k / den, num_g / den
    print(f"{what}: mean-rel error vs fp64 over {len(rows)} rows: kernel {err_k:.4g}, single-pass golden {err_g:.4g}", flush=True)
    assert err_k <= 1.25 * err_g + 1e-4, (what, err_k, err_g)


def test_config2_chain_indexer_then_attention(c_oracle):
    """B=32, KV 8192..65536: the indexer's selection must equal the golden's bit for bit, and the attention
    over it must match the golden within tolerance."""
    B, K = 32, 2048
    lengths = config_lengths(2, seed=2)
    li = gen_indexer_inputs(B, 1, lengths, selected_count=K, seed=2, variant="fp32")
    sfa = gen_sfa_inputs(B, 1, 128, lengths, topk=K, seed=3, block_table=li.block_table, block_num=li.block_num,
                         topk_indices=torch.zeros([B, K], dtype=torch.int32))
    d = li.to(torch.device(DEV))
    pypto_amd.lightning_indexer_decode(d.idx_query, d.idx_query_scale, d.idx_key_cache, d.idx_key_scale, d.idx_weight,
                                       d.act_seq_key, d.block_table, d.topk_res, None, None, K)
    torch.cuda.synchronize()
    want = c_oracle.li_decode(li.idx_query, li.idx_query_scale, li.idx_key_cache, li.idx_key_scale, li.idx_weight,
                              li.act_seq_key, li.block_table, K)
    got = d.topk_res.cpu()
    assert torch.equal(got, want), f"{int((got != want).sum())} index mismatches"
    sel = d.topk_res.reshape(B, K).contiguous()
    out = run_sfa(sfa, topk_indices=sel)
    gold = golden(c_oracle, sfa, topk_indices=sel.cpu())
    check(out, gold, "cfg2 chain")
    assert_close_to_fp64_truth(out, gold, sfa, [(b, 0) for b in (0, 7, 13, 31)], "cfg2 chain", topk_indices=sel.cpu())


def test_config3_two_query_tokens_per_sequence(c_oracle):
    """B=64, S1=2, KV 4096..32768: causal effective lengths, every row against the golden."""
    lengths = config_lengths(3, seed=3)
    inp = gen_sfa_inputs(64, 2, 128, lengths, topk=2048, seed=4)
    out = run_sfa(inp)
    gold = golden(c_oracle, inp)
    check(out, gold, "cfg3")
    assert_close_to_fp64_truth(out, gold, inp, [(0, 0), (0, 1), (21, 1), (63, 0)], "cfg3")


def test_config3_chain_indexer_then_attention(c_oracle):
    """B=64, S1=2, KV 4096..32768, chained at full size: the indexer scores both query tokens of a sequence
    (the first may not select the last position, the second may: eff_seq = act - (S1-1-s)), its indices must
    equal the golden's bit for bit, and the attention over them (cur_seq = min(act - S1 + 1 + s, topk)) must
    match the golden within tolerance."""
    B, S1, K = 64, 2, 2048
    lengths = config_lengths(3, seed=3)
    li = gen_indexer_inputs(B, S1, lengths, selected_count=K, seed=12, variant="fp32")
    sfa = gen_sfa_inputs(B, S1, 128, lengths, topk=K, seed=13, block_table=li.block_table, block_num=li.block_num,
                         topk_indices=torch.zeros([B * S1, K], dtype=torch.int32))
    d = li.to(torch.device(DEV))
    pypto_amd.lightning_indexer_decode(d.idx_query, d.idx_query_scale, d.idx_key_cache, d.idx_key_scale, d.idx_weight,
                                       d.act_seq_key, d.block_table, d.topk_res, None, None, K)
    torch.cuda.synchronize()
    want = c_oracle.li_decode(li.idx_query, li.idx_query_scale, li.idx_key_cache, li.idx_key_scale, li.idx_weight,
                              li.act_seq_key, li.block_table, K)
    got = d.topk_res.cpu()
    assert torch.equal(got, want), f"{int((got != want).sum())} index mismatches"
    # the causal rule, seen in the indices themselves: token 0 of a sequence never holds its last position,
    # token 1 may (and every position is below the token's effective length)
    g = got.reshape(B, S1, K)
    for b, n in enumerate(lengths):
        assert int(g[b, 0].max()) <= n - 2 and int(g[b, 1].max()) <= n - 1
    sel = d.topk_res.reshape(B * S1, K).contiguous()
    out = run_sfa(sfa, topk_indices=sel)
    check(out, golden(c_oracle, sfa, topk_indices=sel.cpu()), "cfg3 chain")


def test_config4_prefill_4096_tokens(c_oracle):
    """B=1, S1=4096, KV 4096: row s sees min(s + 1, 2048) keys.  Every row against the golden; the first
    row, which sees one key, must be that key's de-quantised value row exactly."""
    inp = gen_sfa_inputs(1, 4096, 128, config_lengths(4), topk=2048, seed=5)
    out = run_sfa(inp)
    # row 0: one key (position 0): out = bf16(int8 * scale) of its cache row, for every head
    phys = int(inp.block_table[0, 0]) * inp.block_size
    v = (inp.key_nope_2d[phys].float().reshape(4, 128) * inp.k_nope_scales[phys].reshape(4, 1)).reshape(512)
    v = v.to(torch.bfloat16)
    assert torch.equal(out[0, 0].view(torch.int16), v.view(torch.int16).expand(128, 512)), "single-key row"
    gold = golden(c_oracle, inp)
    check(out, gold, "cfg4")
    # rows that see 2, 100 and 2047 keys, the first with all 2048, a late one and the last
    assert_close_to_fp64_truth(out, gold, inp, [(0, 1), (0, 99), (0, 2046), (0, 2047), (0, 3333), (0, 4095)], "cfg4")


@pytest.mark.parametrize("b,s1,n_q", [(300, 1, 128), (128, 4, 128), (300, 1, 160)])
def test_more_query_rows_than_compute_units(c_oracle, b, s1, n_q):
    """Decode batches past one workgroup per compute unit (the operator's documented range reaches b = 128 with
    s1 = 4, examples/models/deepseek_v32_exp/README.md:6-24): 300 rows, which the library runs as full rounds of
    whole rows plus the rows left over in pieces, and 512 rows; every row against the golden.  160 heads make two
    head groups per row (the second partly filled), so that whole rows and pieces each take two workgroups."""
    act = [2048 + 37 * (i % 11) for i in range(b)]
    inp = gen_sfa_inputs(b, s1, n_q, act, topk=2048, seed=b + s1)
    out = run_sfa(inp)
    gold = golden(c_oracle, inp)
    check(out, gold, f"b={b} s1={s1}")
    assert_close_to_fp64_truth(out, gold, inp, [(0, 0), (b // 2, s1 - 1), (b - 1, 0)], f"b={b} s1={s1}")


def test_prolog_indexer_chain(c_oracle):
    """Prolog -> indexer on the GPU against prolog oracle -> indexer oracle: the prolog's int8 query, fp16 scales
    and weights and its freshly written key rows feed the indexer; the selected indices must be identical."""
    from oracle import lip_oracle as lo
    from pypto_amd.synthetic import gen_indexer_prolog_inputs
    K = 2048
    act = [5000, 4097, 3000, 2049]
    inp = gen_indexer_prolog_inputs(4, 2, act, seed=11)
    inp.q_norm_scale *= 1e-3            # keeps fp16(q_scale * weight) of the indexer finite
    ref = lo.indexer_prolog_ref(*inp.input_tensors())
    t, n = 8, 64
    dev = torch.device(DEV)
    d = inp.to(dev)
    q_int8 = torch.empty([t, n, 128], dtype=torch.int8, device=dev)
    q_scale = torch.empty([t, n, 1], dtype=torch.float16, device=dev)
    weights = torch.empty([t, n], dtype=torch.float16, device=dev)
    pypto_amd.lightning_indexer_prolog_quant(*d.input_tensors(), q_int8, q_scale, d.k_cache, d.k_cache_scale, weights,
                                             pypto_amd.IndexerPrologQuantAttr(), pypto_amd.IndexerPrologQuantConfigs())
    act_t = torch.tensor(act, dtype=torch.int32)
    res = torch.full([t, 1, K], -7, dtype=torch.int32, device=dev)
    nb, bs = d.k_cache.shape[0], d.k_cache.shape[1]
    pypto_amd.lightning_indexer_decode(q_int8, q_scale.reshape(t, n), d.k_cache, d.k_cache_scale.reshape(nb, bs, 1),
                                       weights, act_t.to(dev), d.block_table, res, None, None, K)
    torch.cuda.synchronize()
    want = c_oracle.li_decode(torch.from_numpy(ref["q_int8"]), torch.from_numpy(ref["q_scale"]),
                              torch.from_numpy(ref["k_cache"]), torch.from_numpy(ref["k_cache_scale"]).reshape(nb, bs, 1),
                              torch.from_numpy(ref["weights"]), act_t, inp.block_table, K)
    got = res.cpu()
    assert torch.equal(got, want), f"{int((got != want).sum())} index mismatches"
    # the last two positions of every sequence are the rows the prolog has just written: selectable
    assert int((got >= 0).sum()) == sum(min(a - 1, K) + min(a, K) for a in act)


def test_whole_decode_front_mla_prolog_indexer_prolog_indexer_attention(c_oracle):
    """One decode step of the whole path on the GPU: MLA prolog -> indexer prolog (fed with the MLA prolog's int8
    query latent) -> indexer (over the key rows just written) -> sparse attention (over the latent rows just
    written, with the absorbed query), against the same chain of CPU oracles.  Every intermediate is bit-exact;
    the attention output meets the attention tolerance."""
    from oracle import lip_oracle as lo
    from oracle import mlap_oracle as mo
    from pypto_amd.synthetic import gen_indexer_prolog_inputs, gen_mla_prolog_inputs
    B, S1, K, N = 4, 1, 2048, 128
    act = [5000, 4097, 3000, 2049]
    T = B * S1
    mla = gen_mla_prolog_inputs(B, S1, act, seed=21)
    lip = gen_indexer_prolog_inputs(B, S1, act, seed=22)
    lip.x = mla.token_x                                   # one hidden state feeds both prologs
    # one page table for all caches
    lip.block_table, lip.k_cache_index = mla.block_table, mla.cache_index
    nb, bs = mla.kv_cache.shape[0], mla.kv_cache.shape[1]
    assert lip.k_cache.shape[0] == nb

    # ---- CPU chain
    r_mla = mo.mla_prolog_ref(*mla.input_tensors(), epsilon_cq=1e-5, epsilon_ckv=1e-5)
    lip_args = list(lip.input_tensors())
    lip_args[1] = torch.from_numpy(r_mla["q_norm"])
    lip_args[2] = torch.from_numpy(r_mla["q_norm_scale"]).reshape(T, 1) * 1e-3      # keeps the indexer's fp16 products finite
    r_lip = lo.indexer_prolog_ref(*lip_args)
    act_t = torch.tensor(act, dtype=torch.int32)
    want_idx = c_oracle.li_decode(torch.from_numpy(r_lip["q_int8"]), torch.from_numpy(r_lip["q_scale"]),
                                  torch.from_numpy(r_lip["k_cache"]), torch.from_numpy(r_lip["k_cache_scale"]).reshape(nb, bs, 1),
                                  torch.from_numpy(r_lip["weights"]), act_t, mla.block_table, K)
    qn = torch.from_numpy(r_mla["query_nope"]).to(torch.bfloat16).reshape(T * N, 512)
    qr = torch.from_numpy(r_mla["query_rope"]).to(torch.bfloat16).reshape(T * N, 64)
    kn = torch.from_numpy(r_mla["kv_cache"]).reshape(nb * bs, 512)
    kr = torch.from_numpy(r_mla["kr_cache"]).to(torch.bfloat16).reshape(nb * bs, 64)
    ks = torch.from_numpy(r_mla["k_scale_cache"]).reshape(nb * bs, 4)
    scale = 576 ** -0.5
    want_out = c_oracle.sfa_quant(qn, qr, kn, kr, ks, want_idx.reshape(T, K), mla.block_table, act_t, B, S1, N, K, bs,
                                  scale, s2_tile=0)

    # ---- GPU chain
    dev = torch.device(DEV)
    dm, dl = mla.to(dev), lip.to(dev)
    q_norm = torch.empty([T, 1536], dtype=torch.int8, device=dev)
    q_norm_scale = torch.empty([T, 1], dtype=torch.float32, device=dev)
    q_nope = torch.empty([T, N, 512], dtype=torch.bfloat16, device=dev)
    q_rope = torch.empty([T, N, 64], dtype=torch.bfloat16, device=dev)
    pypto_amd.mla_prolog_quant_d(*dm.input_tensors(), q_norm, q_norm_scale, q_nope, q_rope, dm.kv_cache, dm.kr_cache,
                                 dm.k_scale_cache, 1e-5, 1e-5, "PA_BSND", None, None)
    q_int8 = torch.empty([T, 64, 128], dtype=torch.int8, device=dev)
    q_scale = torch.empty([T, 64, 1], dtype=torch.float16, device=dev)
    weights = torch.empty([T, 64], dtype=torch.float16, device=dev)
    gl = list(dl.input_tensors())
    gl[1], gl[2] = q_norm, q_norm_scale * 1e-3
    pypto_amd.lightning_indexer_prolog_quant(*gl, q_int8, q_scale, dl.k_cache, dl.k_cache_scale, weights)
    res = torch.empty([T, 1, K], dtype=torch.int32, device=dev)
    pypto_amd.lightning_indexer_decode(q_int8, q_scale.reshape(T, 64), dl.k_cache, dl.k_cache_scale.reshape(nb, bs, 1),
                                       weights, act_t.to(dev), dm.block_table, res, None, None, K)
    out = torch.full([B, S1, N, 512], float("nan"), dtype=torch.bfloat16, device=dev)
    pypto_amd.sparse_flash_attention_quant_d(q_nope.reshape(T * N, 512), q_rope.reshape(T * N, 64),
                                             dm.kv_cache.reshape(nb * bs, 512), dm.kr_cache.reshape(nb * bs, 64),
                                             dm.k_scale_cache.reshape(nb * bs, 4), res.reshape(T, K), dm.block_table,
                                             act_t.to(dev), out, N, 1, scale, K, bs, dm.block_table.shape[1], None)
    torch.cuda.synchronize()
    assert torch.equal(q_norm.cpu(), torch.from_numpy(r_mla["q_norm"]))
    assert torch.equal(q_int8.cpu(), torch.from_numpy(r_lip["q_int8"]))
    assert torch.equal(res.cpu(), want_idx), f"{int((res.cpu() != want_idx).sum())} index mismatches"
    check(out.cpu(), want_out, "whole decode front")


# The shapes of the reference's own system-test cases for this operator
# (framework/tests/st/operator/src/test_deepseek_v3.2_exp/gen_gather_selected_attention.py:358-450:
# 128 heads, top-k 2048, blocks of 128; quantized and bf16 latent cache for each), on seeded synthetic data.
@pytest.mark.parametrize("b,s1,act", [
    (4, 2, [65536] * 4),
    (4, 2, [666, 532, 768, 900]),
    (32, 1, [511] * 32),
    (1, 1, [2049]),
    (1, 3, [2047]),
    (128, 1, [8096] * 128),
    (8, 1, [131072] * 8),
    (4, 1, [666, 532, 768, 900]),
    (8, 1, [666, 532, 768, 900, 5698, 2358, 324, 2048]),
])
def test_reference_system_test_shapes(c_oracle, b, s1, act):
    from oracle import sfa_oracle as so
    inp = gen_sfa_inputs(b, s1, 128, act, topk=2048, seed=100 + b + s1)
    out = run_sfa(inp)
    check(out, golden(c_oracle, inp), f"reference case b={b} s1={s1} act={act[0]}..")
    # the bf16-cache branch on exactly the values the int8 cache de-quantises to: the same bits
    d = inp.to(torch.device(DEV))
    kn_bf16 = so.dequant_kn(inp.key_nope_2d, inp.k_nope_scales).to(DEV)
    out_b = torch.full([b, s1, 128, 512], float("nan"), dtype=torch.bfloat16, device=DEV)
    pypto_amd.sparse_flash_attention_quant_d(d.query_nope, d.query_rope, kn_bf16, d.key_rope_2d, None, d.topk_indices,
                                             d.block_table, d.kv_act_seqs, out_b, 128, 1, inp.softmax_scale, 2048,
                                             inp.block_size, inp.max_blocknum_perbatch, None)
    torch.cuda.synchronize()
    assert torch.equal(out_b.cpu().view(torch.int16), out.view(torch.int16))
