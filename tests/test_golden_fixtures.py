"""The committed fixtures under tests/golden/ (inputs + golden outputs, written by
tests/golden/make_fixtures.py): the CPU goldens must still reproduce them bit for bit, the input
generators must still produce the same inputs, and the GPU path is held against them."""
import os

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = os.path.join(HERE, "golden")


def load(name):
    return np.load(os.path.join(GOLD, name), allow_pickle=False)


def t16(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a)).view(dtype)


def sfa_case():
    z = load("sfa_b2_s2_h16_topk64.npz")
    c = dict(query_nope=t16(z["query_nope_bf16"], torch.bfloat16), query_rope=t16(z["query_rope_bf16"], torch.bfloat16),
             key_nope_2d=torch.from_numpy(z["key_nope_2d"]), key_rope_2d=t16(z["key_rope_2d_bf16"], torch.bfloat16),
             k_nope_scales=torch.from_numpy(z["k_nope_scales"]),
             topk_indices=torch.from_numpy(z["topk_indices"]), block_table=torch.from_numpy(z["block_table"]),
             kv_act_seqs=torch.from_numpy(z["kv_act_seqs"]), scale=float(z["softmax_scale"]),
             block_size=int(z["block_size"]), topk=int(z["topk"]), n_q=int(z["n_q"]),
             single=t16(z["out_single_pass_bf16"], torch.bfloat16), online=t16(z["out_online_tile32_bf16"], torch.bfloat16))
    from pypto_amd.synthetic import pack_nope_cache
    c["packed"] = pack_nope_cache(c["key_nope_2d"], c["key_rope_2d"], c["k_nope_scales"])   # layout pinned in test_oracle_sfa.py
    c["b"] = c["kv_act_seqs"].shape[0]
    c["s1"] = c["topk_indices"].shape[0] // c["b"]
    return c


def li_case(variant):
    z = load(f"li_b2_s2_k16_{variant}.npz")
    sdt = torch.float16 if variant == "fp16" else torch.float32
    wdt = torch.float16 if variant == "fp16" else torch.bfloat16
    cvt = lambda a, dt: t16(a, dt) if dt != torch.float32 else torch.from_numpy(a)
    return dict(idx_query=torch.from_numpy(z["idx_query"]), idx_query_scale=cvt(z["idx_query_scale"], sdt),
                idx_key_cache=torch.from_numpy(z["idx_key_cache"]), idx_key_scale=cvt(z["idx_key_scale"], sdt),
                idx_weight=cvt(z["idx_weight"], wdt), act_seq_key=torch.from_numpy(z["act_seq_key"]),
                block_table=torch.from_numpy(z["block_table"]), k=int(z["selected_count"]),
                topk_res=torch.from_numpy(z["topk_res"]))


def test_generators_still_produce_the_fixture_inputs():
    from pypto_amd.synthetic import gen_indexer_inputs, gen_sfa_inputs
    c = sfa_case()
    inp = gen_sfa_inputs(2, 2, 16, [200, 40], topk=64, seed=11)
    assert torch.equal(inp.query_nope.view(torch.int16), c["query_nope"].view(torch.int16))
    assert torch.equal(inp.key_nope_2d, c["key_nope_2d"]) and torch.equal(inp.topk_indices, c["topk_indices"])
    assert torch.equal(inp.block_table, c["block_table"])
    for variant in ("fp16", "fp32"):
        f = li_case(variant)
        li = gen_indexer_inputs(2, 2, [300, 40], selected_count=16, seed=12, variant=variant)
        assert torch.equal(li.idx_query, f["idx_query"]) and torch.equal(li.idx_key_cache, f["idx_key_cache"])
        assert torch.equal(li.block_table, f["block_table"])


def test_cpu_goldens_reproduce_the_fixtures(c_oracle):
    from oracle import li_oracle, sfa_oracle
    c = sfa_case()
    q = torch.cat([c["query_nope"], c["query_rope"]], dim=-1).reshape(c["b"], c["s1"], c["n_q"], 576)
    act = c["kv_act_seqs"].tolist()
    args = (q, c["key_nope_2d"], c["key_rope_2d"], c["k_nope_scales"], c["topk_indices"], c["block_table"], act,
            c["block_size"], c["scale"], c["topk"])
    assert torch.equal(sfa_oracle.sfa_single_pass(*args).view(torch.int16), c["single"].view(torch.int16))
    assert torch.equal(sfa_oracle.sfa_online(*args, s2_tile=32).view(torch.int16), c["online"].view(torch.int16))
    packed = sfa_oracle.sa_antiquant_single_pass(q, c["packed"], c["topk_indices"], c["block_table"], act,
                                                 c["block_size"], c["scale"], c["topk"])
    assert torch.equal(packed.view(torch.int16), c["single"].view(torch.int16))
    for variant in ("fp16", "fp32"):
        f = li_case(variant)
        a = (f["idx_query"], f["idx_query_scale"], f["idx_key_cache"], f["idx_key_scale"], f["idx_weight"],
             f["act_seq_key"], f["block_table"], f["k"])
        assert torch.equal(li_oracle.lightning_indexer_ref(*a), f["topk_res"])
        assert torch.equal(c_oracle.li_decode(*a), f["topk_res"])


@pytest.mark.gpu
def test_gpu_path_against_the_fixtures():
    import pypto_amd
    from pypto_amd.utils import attention_error_stats
    dev = torch.device("cuda:0")
    c = sfa_case()
    out = torch.full([c["b"], c["s1"], c["n_q"], 512], float("nan"), dtype=torch.bfloat16, device=dev)
    g = {k: v.to(dev) for k, v in c.items() if isinstance(v, torch.Tensor)}
    pypto_amd.sparse_flash_attention_quant_d(g["query_nope"], g["query_rope"], g["key_nope_2d"], g["key_rope_2d"],
                                             g["k_nope_scales"], g["topk_indices"], g["block_table"], g["kv_act_seqs"],
                                             out, c["n_q"], 1, c["scale"], c["topk"], c["block_size"],
                                             g["block_table"].shape[1], None)
    out_p = torch.full_like(out, float("nan"))
    pypto_amd.sparse_attention_antiquant_d(g["query_nope"], g["query_rope"], g["packed"], g["topk_indices"],
                                           g["block_table"], g["kv_act_seqs"], out_p, c["n_q"], 1, c["scale"], c["topk"],
                                           c["block_size"], g["block_table"].shape[1], None)
    torch.cuda.synchronize()
    for o in (out.cpu(), out_p.cpu()):
        max_abs, mean_rel = attention_error_stats(o, c["single"])     # tolerance: max-abs 2e-2, mean-rel 5e-3
        assert max_abs <= 2e-2 and mean_rel <= 5e-3, (max_abs, mean_rel)
    for variant in ("fp16", "fp32"):
        f = li_case(variant)
        d = {k: v.to(dev) for k, v in f.items() if isinstance(v, torch.Tensor)}
        res = torch.full_like(d["topk_res"], -7)
        pypto_amd.lightning_indexer_decode(d["idx_query"], d["idx_query_scale"], d["idx_key_cache"], d["idx_key_scale"],
                                           d["idx_weight"], d["act_seq_key"], d["block_table"], res, None, None, f["k"])
        torch.cuda.synchronize()
        assert torch.equal(res.cpu(), f["topk_res"]), variant
