"""The operators under HIP graph capture: a serving loop records indexer -> attention once and replays it.
Every replay, with inputs changed in place between replays and eager work of the same operators in between,
must give exactly what the eager calls give on the same inputs (same kernels, so bit for bit)."""
import pytest
import torch

import pypto_amd
from pypto_amd.synthetic import gen_indexer_inputs, gen_sfa_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _chain(li, sfa, out, k):
    pypto_amd.lightning_indexer_decode(li.idx_query, li.idx_query_scale, li.idx_key_cache, li.idx_key_scale, li.idx_weight,
                                       li.act_seq_key, li.block_table, li.topk_res, None, None, k)
    sel = li.topk_res.reshape(li.topk_res.shape[0], k)
    pypto_amd.sparse_flash_attention_quant_d(sfa.query_nope, sfa.query_rope, sfa.key_nope_2d, sfa.key_rope_2d,
                                             sfa.k_nope_scales, sel, sfa.block_table, sfa.kv_act_seqs, out, 128, 1,
                                             sfa.softmax_scale, k, 128, sfa.max_blocknum_perbatch, None)


def test_indexer_then_attention_replays_match_eager():
    b, k = 8, 2048
    act = [9000, 4097, 2049, 2048, 700, 31, 12000, 5000]
    li_h = gen_indexer_inputs(b, 1, act, selected_count=k, seed=11, variant="fp32")
    sfa_h = gen_sfa_inputs(b, 1, 128, act, topk=k, seed=12, block_table=li_h.block_table, block_num=li_h.block_num,
                           topk_indices=torch.zeros([b, k], dtype=torch.int32))
    dev = torch.device(DEV)
    li, sfa = li_h.to(dev), sfa_h.to(dev)
    out_g = torch.zeros([b, 1, 128, 512], dtype=torch.bfloat16, device=dev)
    out_e = torch.zeros_like(out_g)

    # warm-up on a side stream (allocator pools, lazy initialisation), then capture
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        _chain(li, sfa, out_g, k)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _chain(li, sfa, out_g, k)

    gen = torch.Generator().manual_seed(5)
    for rep in range(4):
        # new queries in place: other scores, another selection, other attention inputs
        li.idx_query.copy_(torch.randint(-127, 128, li.idx_query.shape, generator=gen, dtype=torch.int8))
        sfa.query_nope.copy_(torch.randn(sfa.query_nope.shape, generator=gen).to(torch.bfloat16))
        out_g.fill_(float("nan"))
        li.topk_res.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        got_sel, got = li.topk_res.clone(), out_g.clone()
        # the same through eager calls (which also stand for the program's own work between replays)
        li.topk_res.fill_(-7)
        _chain(li, sfa, out_e, k)
        torch.cuda.synchronize()
        assert torch.equal(got_sel, li.topk_res), f"replay {rep}: selection differs from the eager call"
        assert not torch.isnan(got).any(), f"replay {rep}: NaN"
        assert torch.equal(got.view(torch.int16), out_e.view(torch.int16)), f"replay {rep}: attention differs"


@pytest.mark.parametrize("b,s1,act,ni", [(4, 2, [5000, 300, 129, 64], 4),      # decode kernels
                                         (3, 50, [700, 650, 600], 8)])         # 150 tokens: the prefill forms of every stage
def test_prologs_replays_match_eager(b, s1, act, ni):
    """MLA prolog + indexer prolog recorded once; hidden states change in place between replays, the caches start
    from the same state each time."""
    from pypto_amd.synthetic import gen_indexer_prolog_inputs, gen_mla_prolog_inputs
    dev = torch.device(DEV)
    kw = dict(h=512, q_lora_rank=1536)
    mla = gen_mla_prolog_inputs(b, s1, act, seed=21, n_heads=8, **kw).to(dev)
    lip = gen_indexer_prolog_inputs(b, s1, act, seed=22, n_heads=ni, **kw).to(dev)
    t = b * s1
    caches = [mla.kv_cache, mla.kr_cache, mla.k_scale_cache, lip.k_cache, lip.k_cache_scale]
    base = [c.clone() for c in caches]

    def outputs():
        return (torch.zeros(t, 1536, dtype=torch.int8, device=dev), torch.zeros(t, 1, device=dev),
                torch.zeros(t, 8, 512, dtype=torch.bfloat16, device=dev), torch.zeros(t, 8, 64, dtype=torch.bfloat16, device=dev),
                torch.zeros(t, ni, 128, dtype=torch.int8, device=dev), torch.zeros(t, ni, 1, dtype=torch.float16, device=dev),
                torch.zeros(t, ni, dtype=torch.float16, device=dev))

    def run(o):
        qn, qs, qnope, qrope, iq, iqs, iw = o
        pypto_amd.mla_prolog_quant_d(*mla.input_tensors(), qn, qs, qnope, qrope, mla.kv_cache, mla.kr_cache,
                                     mla.k_scale_cache, 1e-5, 1e-5, "PA_BSND", None, None)
        ins = list(lip.input_tensors())
        ins[0], ins[1], ins[2] = mla.token_x, qn, qs            # hidden states, query latent and its scale chained
        pypto_amd.lightning_indexer_prolog_quant(*ins, iq, iqs, lip.k_cache, lip.k_cache_scale, iw)

    o_g, o_e = outputs(), outputs()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        run(o_g)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(o_g)
    gen = torch.Generator().manual_seed(9)
    for rep in range(3):
        mla.token_x.copy_(torch.randn(mla.token_x.shape, generator=gen).to(torch.bfloat16))
        for c, b0 in zip(caches, base):
            c.copy_(b0)
        graph.replay()
        torch.cuda.synchronize()
        got = [x.clone() for x in o_g] + [c.clone() for c in caches]
        for c, b0 in zip(caches, base):
            c.copy_(b0)
        run(o_e)
        torch.cuda.synchronize()
        want = list(o_e) + caches
        for i, (g_, w_) in enumerate(zip(got, want)):
            assert torch.equal(g_.view(torch.uint8), w_.view(torch.uint8)), f"replay {rep}: output {i} differs from the eager call"


@pytest.mark.parametrize("b,s1,act", [(4, 2, [5000, 300, 129, 64]), (16, 2, [5000, 300, 129, 64] * 4)])
def test_fused_prolog_operator_replays_match_the_two_operators_called_eagerly(b, s1, act):
    """mla_indexer_prolog_quant_d (one library call, one workspace from torch's pool, the last launches of the two
    halves merged) recorded once and replayed with new hidden states: every replay equals the two separate
    operators called eagerly on the same inputs, bit for bit.  8 tokens: the decode forms' four launches; 32 tokens:
    the MLA half's matrix-core forms with the indexer half's first launch riding in them."""
    from pypto_amd.synthetic import gen_indexer_prolog_inputs, gen_mla_prolog_inputs
    dev = torch.device(DEV)
    kw = dict(h=512, q_lora_rank=1536)
    mla = gen_mla_prolog_inputs(b, s1, act, seed=31, n_heads=8, **kw).to(dev)
    lip = gen_indexer_prolog_inputs(b, s1, act, seed=32, n_heads=4, **kw).to(dev)
    t = b * s1
    caches = [mla.kv_cache, mla.kr_cache, mla.k_scale_cache, lip.k_cache, lip.k_cache_scale]
    base = [c.clone() for c in caches]

    def outputs():
        return (torch.zeros(t, 8, 512, dtype=torch.bfloat16, device=dev), torch.zeros(t, 8, 64, dtype=torch.bfloat16, device=dev),
                torch.zeros(t, 4, 128, dtype=torch.int8, device=dev), torch.zeros(t, 4, 1, dtype=torch.float16, device=dev),
                torch.zeros(t, 4, dtype=torch.float16, device=dev))

    def fused(o):
        qnope, qrope, iq, iqs, iw = o
        pypto_amd.mla_indexer_prolog_quant_d(
            mla.token_x, mla.w_dq, mla.w_uq_qr, mla.dequant_scale, mla.w_uk, mla.w_dkv_kr, mla.gamma_cq, mla.gamma_ckv, mla.cos,
            mla.sin, mla.cache_index, mla.kv_cache, mla.kr_cache, mla.k_scale_cache, lip.w_qb, lip.w_qb_scale, lip.wk, lip.w_proj,
            lip.ln_gamma_k, lip.ln_beta_k, lip.hadamard_q, lip.hadamard_k, lip.k_cache, lip.k_cache_scale, qnope, qrope,
            mla.kv_cache, mla.kr_cache, mla.k_scale_cache, iq, iqs, lip.k_cache, lip.k_cache_scale, iw, 1e-5, 1e-5, "PA_BSND",
            None, None, None, None)

    def separate(o):
        qnope, qrope, iq, iqs, iw = o
        qn = torch.zeros(t, 1536, dtype=torch.int8, device=dev)
        qs = torch.zeros(t, 1, device=dev)
        pypto_amd.mla_prolog_quant_d(mla.token_x, mla.w_dq, mla.w_uq_qr, mla.dequant_scale, mla.w_uk, mla.w_dkv_kr, mla.gamma_cq,
                                     mla.gamma_ckv, mla.cos, mla.sin, mla.cache_index, mla.kv_cache, mla.kr_cache,
                                     mla.k_scale_cache, qn, qs, qnope, qrope, mla.kv_cache, mla.kr_cache, mla.k_scale_cache,
                                     1e-5, 1e-5, "PA_BSND", None, None)
        pypto_amd.lightning_indexer_prolog_quant(mla.token_x, qn, qs, lip.w_qb, lip.w_qb_scale, lip.wk, lip.w_proj, lip.ln_gamma_k,
                                                 lip.ln_beta_k, mla.cos, mla.sin, lip.hadamard_q, lip.hadamard_k, lip.k_cache,
                                                 lip.k_cache_scale, mla.cache_index, iq, iqs, lip.k_cache, lip.k_cache_scale, iw)

    o_g, o_e = outputs(), outputs()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        fused(o_g)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fused(o_g)
    gen = torch.Generator().manual_seed(19)
    for rep in range(3):
        mla.token_x.copy_(torch.randn(mla.token_x.shape, generator=gen).to(torch.bfloat16))
        for c, b0 in zip(caches, base):
            c.copy_(b0)
        graph.replay()
        torch.cuda.synchronize()
        got = [x.clone() for x in o_g] + [c.clone() for c in caches]
        for c, b0 in zip(caches, base):
            c.copy_(b0)
        separate(o_e)
        torch.cuda.synchronize()
        want = list(o_e) + caches
        for i, (g_, w_) in enumerate(zip(got, want)):
            assert torch.equal(g_.view(torch.uint8), w_.view(torch.uint8)), f"replay {rep}: output {i} differs from the separate operators"
