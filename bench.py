#!/usr/bin/env python3
"""Benchmark of the quantized DeepSeek-V3.2 sparse-attention decode path on one MI355X.

A step is one pass of sparse flash attention over one batch: B=32 sequences, one query token each,
128 heads, d=576/512, top-k 2048 chosen by the lightning indexer, paged int8 latent KV with per-token
scales, per-sequence KV lengths drawn from 8192..65536.  All inputs are resident in HBM before the
timed region.  Prints ONE JSON line:

  value          query tokens per second (B / step time) over K timed steps, after SETTLE_STEPS untimed steps
                 ("ms_per_step_unsettled": the same K steps timed before them, after the caller's warm-up only)
  roofline       achieved bf16 matrix throughput of the attention launch = algorithmic flops per step
                 / average launch duration from HIP events on the launch stream, against 2.5 PFLOP/s;
                 the HBM-side figure (algorithmic bytes / same duration, against 8 TB/s) is in
                 "roofline_hbm" because the shape sits at the ridge of the two
  packed_cache   the same step through sparse_attention_antiquant_d (one 656-byte row per key)
  indexer        time of one lightning-indexer pass (score + select) on the same batch, on the
                 indexer-only configuration (B=4, KV 32768) and on configs[3]'s batch (B=64, two query
                 tokens per sequence), with its HBM fraction and the counter-derived HBM traffic
  indexer_prolog time of one lightning-indexer prolog pass (projection stage) on the reference's enabled
                 case b=4, s1=2 (8 tokens, h=7168, q_lora_rank=1536), launches replayed from a HIP graph so
                 that host time between launches is not counted, with its HBM fraction
  mla_prolog     the same for the MLA prolog (b=4, s=2, 128 heads; 85 MB of weights per pass, ten sets);
                 all three prolog legs also carry "batch_of_32": the same pass at the headline's 32 tokens
  cpu_baseline   the scalar C statement of the golden, all host threads, on a bounded sample of the
                 same batch; beside it the torch golden at configs[0] in its literal loop form and vectorised

To keep a step from being served out of the 256 MB memory-side cache, steps rotate over ROT
different selections (different indexer queries over the same caches).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0
ROT = 8
SETTLE_STEPS = 1000   # untimed attention steps ahead of the caller's warm-up: about 40 ms of load, see main()
COPY_MIB = 256
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "sfa_decode_cfg2_hbm_traffic.md")
LI_TRAFFIC_FILE = os.path.join(ROOT, "profiles", "indexer_hbm_traffic.md")


def measured_traffic(path, key, library_version, expect=None):
    """HBM bytes per launch from a committed counter summary under profiles/ (FETCH_SIZE and WRITE_SIZE of the
    kernels, scaled by what the same counters read for a device copy of known size): the line '<key>: N'.
    The summary names the library version it was taken with ('library_version: x.y.z') and may name other
    launch facts ('<name>: value' lines listed in `expect`); when any of them no longer matches the built
    library the figure is stale and None is returned instead."""
    try:
        fields = {}
        with open(path) as f:
            for ln in f:
                m = ln.strip().split(":", 1)
                if len(m) == 2 and " " not in m[0]:
                    fields[m[0]] = m[1].strip()
    except OSError:
        return None
    if fields.get("library_version") != library_version or key not in fields:
        return None
    for name, want in (expect or {}).items():
        if fields.get(name) != str(want):
            return None
    try:
        return int(fields[key])
    except ValueError:
        return None


def sfa_algorithmic_work(cur_seqs, n_heads=128):
    """Bytes and flops of one step: per query row with n selected keys,
    n*(512 + 128 + 16) KV + n*4 indices + 4 per page touched (<= n, counted as min(n, pages)) +
    heads*576*2 query + heads*512*2 output; flops = 2*heads*n*(576+512)."""
    byt = flops = 0
    for n in cur_seqs:
        byt += n * (512 + 128 + 16) + n * 4 + 4 * n + n_heads * 576 * 2 + n_heads * 512 * 2
        flops += 2 * n_heads * n * (576 + 512)
    return byt, flops


def indexer_algorithmic_bytes(lengths, k_scale_bytes, k=2048):
    """Per query token over L keys: L*(128 + scale) + 64*128 query + 64*(scale+weight) + 4 per page + k*4 out."""
    return sum(L * (128 + k_scale_bytes) + 64 * 128 + 64 * 8 + 4 * math.ceil(L / 128) + k * 4 for L in lengths)


def time_events(fn, steps, warmup, torch):
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for i, (a, b) in enumerate(evs):
        a.record()
        fn(warmup + i)
        b.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per = [a.elapsed_time(b) for a, b in evs]            # ms, device time of the launches of one step
    return wall, sum(per) / len(per), min(per)


def time_batch(fn, steps, warmup, torch):
    """Average device time per step of `steps` back-to-back steps: one HIP event pair around the whole batch
    (no host synchronisation and no event between the steps, as the steps of a decode loop follow one another)."""
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for i in range(steps):
        fn(warmup + i)
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / steps


def prolog_leg(torch, dev, pypto_amd, b=4, s1=2, calls=20, replays=10):
    """One prolog pass = both launches of lightning_indexer_prolog_quant.  `calls` passes are captured
    into a HIP graph (the operator allocates its workspace from torch's pool, which capture supports)
    and the graph is replayed; falls back to timing eager calls if capture is unavailable."""
    from pypto_amd.synthetic import gen_indexer_prolog_inputs
    d = gen_indexer_prolog_inputs(b, s1, [65536] * b, seed=0).to(dev)
    t, n = b * s1, d.w_proj.shape[1]
    outs = (torch.empty([t, n, 128], dtype=torch.int8, device=dev), torch.empty([t, n, 1], dtype=torch.float16, device=dev),
            d.k_cache, d.k_cache_scale, torch.empty([t, n], dtype=torch.float16, device=dev))

    # every captured pass reads its own copy of the three weight matrices (20 x 15.3 MB > the 256 MB
    # memory-side cache), as a layer's weights are cold when its turn comes in a real decode step
    ins = list(d.input_tensors())
    sets = [(ins[3].clone(), ins[5].clone(), ins[6].clone()) for _ in range(calls)]

    def one(i=0):
        a = list(ins)
        a[3], a[5], a[6] = sets[i]
        pypto_amd.lightning_indexer_prolog_quant(*a, *outs)
    for _ in range(3):
        one()
    torch.cuda.synchronize()
    mode = "hip graph replay"
    try:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(calls):
                one(i)
        run = g.replay
    except Exception:                      # noqa: BLE001 -- capture support varies; eager timing still valid
        mode = "eager calls (host time included)"

        def run():
            for i in range(calls):
                one(i)
    run()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(replays):
        run()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / (calls * replays)
    h, ql = d.x.shape[1], d.q_norm.shape[1]
    byt = ql * n * 128 + h * 128 * 2 + h * n * 2 + 2 * 128 * 128 * 2 + t * (h * 2 + ql + n * 128 + n * 4 + 128 + 2 + 2 * 128)
    return {"workload": f"b={b} s1={s1} (t={t}) h={h} q_lora_rank={ql} {n} heads", "us_per_pass": us, "timing": mode + f", {calls} weight sets in rotation",
            "bytes": byt, "hbm_frac": byt / (us * 1e-6) / 1e9 / PEAK_HBM_GBS}


def mla_prolog_leg(torch, dev, pypto_amd, b=4, s1=2, calls=10, replays=10):
    """One MLA prolog pass = the four launches of mla_prolog_quant_d; timed like prolog_leg (HIP graph of `calls`
    passes, each with its own copy of the four weight tensors: 10 x 85 MB exceeds the memory-side cache)."""
    from pypto_amd.synthetic import gen_mla_prolog_inputs
    d = gen_mla_prolog_inputs(b, s1, [4096] * b, seed=0).to(dev)
    t, n, ql, h = b * s1, d.w_uk.shape[0], d.w_dq.shape[1], d.token_x.shape[1]
    outs = (torch.empty([t, ql], dtype=torch.int8, device=dev), torch.empty([t, 1], dtype=torch.float32, device=dev),
            torch.empty([t, n, 512], dtype=torch.bfloat16, device=dev), torch.empty([t, n, 64], dtype=torch.bfloat16, device=dev),
            d.kv_cache, d.kr_cache, d.k_scale_cache)
    ins = list(d.input_tensors())
    sets = [(ins[1].clone(), ins[2].clone(), ins[4].clone(), ins[5].clone()) for _ in range(calls)]

    def one(i=0):
        a = list(ins)
        a[1], a[2], a[4], a[5] = sets[i]
        pypto_amd.mla_prolog_quant_d(*a, *outs, 1e-5, 1e-5, "PA_BSND", None, None)
    for _ in range(3):
        one()
    torch.cuda.synchronize()
    mode = "hip graph replay"
    try:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(calls):
                one(i)
        run = g.replay
    except Exception:                      # noqa: BLE001 -- capture support varies; eager timing still valid
        mode = "eager calls (host time included)"

        def run():
            for i in range(calls):
                one(i)
    run()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(replays):
        run()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / (calls * replays)
    byt = h * ql * 2 + ql * n * 192 + n * 128 * 512 * 2 + h * 576 * 2 + t * (h * 2 + ql + n * 576 * 2 + 656)
    return {"workload": f"b={b} s={s1} (t={t}) h={h} q_lora_rank={ql} {n} heads", "us_per_pass": us,
            "timing": mode + f", {calls} weight sets in rotation", "bytes": byt,
            "hbm_frac": byt / (us * 1e-6) / 1e9 / PEAK_HBM_GBS}


def fused_prolog_leg(torch, dev, pypto_amd, b=4, s1=2, calls=10, replays=10):
    """One pass of mla_indexer_prolog_quant_d (MLA prolog, then the indexer prolog on its query latent), timed
    like the two legs above: a HIP graph of `calls` passes, each with its own copy of all seven weight tensors."""
    from pypto_amd.synthetic import gen_indexer_prolog_inputs, gen_mla_prolog_inputs
    m = gen_mla_prolog_inputs(b, s1, [4096] * b, seed=0).to(dev)
    ip = gen_indexer_prolog_inputs(b, s1, [4096] * b, seed=0).to(dev)
    t, n, ql = b * s1, m.w_uk.shape[0], m.w_dq.shape[1]
    ni = ip.w_proj.shape[1]
    outs_m = (torch.empty([t, n, 512], dtype=torch.bfloat16, device=dev), torch.empty([t, n, 64], dtype=torch.bfloat16, device=dev),
              m.kv_cache, m.kr_cache, m.k_scale_cache)
    outs_i = (torch.empty([t, ni, 128], dtype=torch.int8, device=dev), torch.empty([t, ni, 1], dtype=torch.float16, device=dev),
              ip.k_cache, ip.k_cache_scale, torch.empty([t, ni], dtype=torch.float16, device=dev))
    sets = [(m.w_dq.clone(), m.w_uq_qr.clone(), m.w_uk.clone(), m.w_dkv_kr.clone(), ip.w_qb.clone(), ip.wk.clone(),
             ip.w_proj.clone()) for _ in range(calls)]

    def one(i=0):
        wdq, wuq, wuk, wdkv, wqb, wk, wproj = sets[i]
        pypto_amd.mla_indexer_prolog_quant_d(
            m.token_x, wdq, wuq, m.dequant_scale, wuk, wdkv, m.gamma_cq, m.gamma_ckv, m.cos, m.sin, m.cache_index,
            m.kv_cache, m.kr_cache, m.k_scale_cache, wqb, ip.w_qb_scale, wk, wproj, ip.ln_gamma_k, ip.ln_beta_k,
            ip.hadamard_q, ip.hadamard_k, ip.k_cache, ip.k_cache_scale, *outs_m, *outs_i, 1e-5, 1e-5, "PA_BSND", None,
            None, None, None)
    for _ in range(3):
        one()
    torch.cuda.synchronize()
    mode = "hip graph replay"
    try:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(calls):
                one(i)
        run = g.replay
    except Exception:                      # noqa: BLE001 -- capture support varies; eager timing still valid
        mode = "eager calls (host time included)"

        def run():
            for i in range(calls):
                one(i)
    run()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(replays):
        run()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / (calls * replays)
    return {"workload": f"b={b} s={s1} (t={t}) MLA prolog ({n} heads) + indexer prolog ({ni} heads)", "us_per_pass": us,
            "timing": mode + f", {calls} weight sets in rotation"}


def other_shapes_leg(torch, pypto_amd, dev):
    """configs[3] and configs[4] through the same operators (parity of both is a GPU test): step time and the
    fraction of the dense bf16 peak their algorithmic flops reach.  Row (b, s) attends
    min(max(act[b] - S1 + 1 + s, 0), 2048) keys."""
    from pypto_amd.synthetic import config_lengths, gen_sfa_inputs
    res = []
    for name, b, s1, lengths, entry, steps in (
            ("configs[3]: B=64 S_q=2 KV 4096-32768", 64, 2, config_lengths(3, seed=3), "d", 200),
            ("configs[4]: B=1 S_q=4096 KV 4096 (row t sees min(t+1, 2048) keys)", 1, 4096, config_lengths(4), "p", 20)):
        inp = gen_sfa_inputs(b, s1, 128, lengths, topk=2048, seed=5).to(dev)
        out = torch.empty([b, s1, 128, 512], dtype=torch.bfloat16, device=dev)
        fn = pypto_amd.sparse_flash_attention_quant_d if entry == "d" else pypto_amd.sparse_flash_attention_quant_p

        def step():
            fn(inp.query_nope, inp.query_rope, inp.key_nope_2d, inp.key_rope_2d, inp.k_nope_scales, inp.topk_indices,
               inp.block_table, inp.kv_act_seqs, out, 128, 1, inp.softmax_scale, 2048, 128, inp.max_blocknum_perbatch, None)
        # the device raises its clocks over the first tens of milliseconds of load: 0.3 s of untimed steps first
        t_settle = time.perf_counter()
        while time.perf_counter() - t_settle < 0.3:
            for _ in range(10):
                step()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            step()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        keys = sum(min(max(int(lengths[bi]) - s1 + 1 + si, 0), 2048) for bi in range(b) for si in range(s1))
        flops = 2.0 * 128 * keys * 1088
        res.append({"workload": name, "us_per_step": ms * 1e3, "tokens_per_s": b * s1 / (ms * 1e-3),
                    "tflops": flops / (ms * 1e-3) / 1e12, "mfma_frac": flops / (ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS})
        del inp, out
    return res


def prefill_prologs_leg(torch, pypto_amd, dev):
    """The two prologs at the reference's prefill-sized cases (MLA prolog b=1 s=512; indexer prolog b=128 s=4 and
    b=1 s=4096) and the MLA prolog at a decode batch of 32: time per eager call, in the default summation mode,
    with every sum of the MLA prolog in its fixed order, and with the indexer's sums over the hidden axis on the
    matrix cores."""
    from pypto_amd import lightning_indexer_prolog_quant_impl as lip_impl
    from pypto_amd.synthetic import gen_indexer_prolog_inputs, gen_mla_prolog_inputs

    def timed(fn, n=20):
        t_settle = time.perf_counter()                  # 0.3 s of untimed calls: the device clocks rise under load
        while time.perf_counter() - t_settle < 0.3:
            for _ in range(5):
                fn()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n * 1e3
    res = []
    from pypto_amd import mla_prolog_quant_impl as mla_impl
    # the MLA prolog at the batch of configs[2] (32 sequences, one token each) in both summation modes -- the default
    # takes the prefill forms from 9 tokens on, the exact mode keeps the decode forms up to 63 -- and at 512 tokens
    for b, s1, exact in ((32, 1, False), (32, 1, True), (1, 512, False)):
        d = gen_mla_prolog_inputs(b, s1, [4096] * b, seed=0).to(dev)
        t, n, ql = b * s1, 128, 1536
        outs = (torch.empty([t, ql], dtype=torch.int8, device=dev), torch.empty([t, 1], dtype=torch.float32, device=dev),
                torch.empty([t, n, 512], dtype=torch.bfloat16, device=dev), torch.empty([t, n, 64], dtype=torch.bfloat16, device=dev),
                d.kv_cache, d.kr_cache, d.k_scale_cache)
        ins = list(d.input_tensors())
        mla_impl.EXACT_ABSORB = exact
        try:
            us = timed(lambda: pypto_amd.mla_prolog_quant_p(*ins, *outs, 1e-5, 1e-5, "PA_BSND", None, None))
        finally:
            mla_impl.EXACT_ABSORB = False
        res.append({"operator": "mla_prolog_quant_p", "tokens": t, "sums": "every sum in its fixed order" if exact else "default", "us_per_call": us})
        del d, outs, ins
    for b, s1, act in ((128, 4, [8192] * 128), (1, 4096, [65536])):
        d = gen_indexer_prolog_inputs(b, s1, act, seed=0).to(dev)
        t, n = b * s1, d.w_proj.shape[1]
        outs = (torch.empty([t, n, 128], dtype=torch.int8, device=dev), torch.empty([t, n, 1], dtype=torch.float16, device=dev),
                d.k_cache, d.k_cache_scale, torch.empty([t, n], dtype=torch.float16, device=dev))
        ins = list(d.input_tensors())
        for mode in ("default", "hidden-axis sums on the matrix cores"):
            lip_impl.MATRIX_CORE_HIDDEN_SUMS = mode != "default"
            try:
                us = timed(lambda: pypto_amd.lightning_indexer_prolog_quant(*ins, *outs))
            finally:
                lip_impl.MATRIX_CORE_HIDDEN_SUMS = False
            res.append({"operator": "lightning_indexer_prolog_quant", "tokens": t, "sums": mode, "us_per_call": us})
        del d, outs, ins
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=200)    # the device clocks settle over the first ~200 steps
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--counter-run", action="store_true",
                    help="for rocprofv3 --pmc: a few attention steps plus one device copy of COPY_MIB MiB "
                         "(the calibration kernel of the counters), no timing, no JSON line")
    ap.add_argument("--seed", type=int, default=2)
    ap.add_argument("--other-shapes", action="store_true",
                    help="also time configs[3] (B=64, two query tokens) and configs[4] (4096-token prefill chunk) "
                         "and add them to the JSON line as 'other_shapes'")
    ap.add_argument("--prefill-prologs", action="store_true",
                    help="also time the MLA prolog at 512 tokens and the indexer prolog at 512 and 4096 tokens "
                         "and add them to the JSON line as 'prefill_prologs'")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path is built and measured on ONE GPU; run with --gpus 1 "
              "(query rows shard over GPUs without any exchange; that is not implemented here)", file=sys.stderr)
        sys.exit(2)

    import torch

    import pypto_amd
    from pypto_amd.synthetic import config_lengths, gen_indexer_inputs, gen_sfa_inputs

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    # ------------------------------------------------------------------ inputs (configuration 2)
    B, S1, NQ, K = 32, 1, 128, 2048
    lengths = config_lengths(2, seed=args.seed)
    li = gen_indexer_inputs(B, S1, lengths, selected_count=K, seed=args.seed, variant="fp32")
    sfa = gen_sfa_inputs(B, S1, NQ, lengths, topk=K, seed=args.seed + 1, block_table=li.block_table,
                         block_num=li.block_num, topk_indices=torch.zeros([B, K], dtype=torch.int32))
    li_d, sfa_d = li.to(dev), sfa.to(dev)

    # ROT selections: the indexer run on ROT different query sets over the same key cache
    g = torch.Generator().manual_seed(args.seed + 77)
    sel = []
    idx_queries = []
    for r in range(ROT):
        q = li.idx_query if r == 0 else torch.randint(-127, 128, li.idx_query.shape, generator=g, dtype=torch.int8)
        qd = q.to(dev)
        idx_queries.append(qd)
        res = torch.empty([B, 1, K], dtype=torch.int32, device=dev)
        pypto_amd.lightning_indexer_decode(qd, li_d.idx_query_scale, li_d.idx_key_cache, li_d.idx_key_scale,
                                           li_d.idx_weight, li_d.act_seq_key, li_d.block_table, res, None, None, K)
        sel.append(res.reshape(B, K).contiguous())
    torch.cuda.synchronize()
    out = torch.zeros([B, S1, NQ, 512], dtype=torch.bfloat16, device=dev)

    def sfa_step(i):
        pypto_amd.sparse_flash_attention_quant_d(sfa_d.query_nope, sfa_d.query_rope, sfa_d.key_nope_2d,
                                                 sfa_d.key_rope_2d, sfa_d.k_nope_scales, sel[i % ROT],
                                                 sfa_d.block_table, sfa_d.kv_act_seqs, out, NQ, 1,
                                                 sfa.softmax_scale, K, 128, sfa.max_blocknum_perbatch, None)

    if args.counter_run:
        for i in range(2 * ROT):
            sfa_step(i)
        # the indexer on the same batch and on configs[1], for its kernels' counters
        res_c = torch.empty([B, 1, K], dtype=torch.int32, device=dev)
        li1_c = gen_indexer_inputs(4, 1, config_lengths(1), selected_count=K, seed=1, variant="fp32").to(dev)
        for i in range(ROT):
            pypto_amd.lightning_indexer_decode(idx_queries[i], li_d.idx_query_scale, li_d.idx_key_cache, li_d.idx_key_scale,
                                               li_d.idx_weight, li_d.act_seq_key, li_d.block_table, res_c, None, None, K)
            pypto_amd.lightning_indexer_decode(li1_c.idx_query, li1_c.idx_query_scale, li1_c.idx_key_cache,
                                               li1_c.idx_key_scale, li1_c.idx_weight, li1_c.act_seq_key, li1_c.block_table,
                                               li1_c.topk_res, None, None, K)
        src = torch.empty(COPY_MIB << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        return

    # ------------------------------------------------------------------ timed region (attention)
    # The device raises its clocks over the first tens of milliseconds of load: by the event pair below the same
    # 20 steps take 41.1-42.0 us each after 5 or 255 earlier steps and 38.5-39.1 us after 1000 or 4000.  A
    # decode loop runs for seconds, so the step is timed at the settled clocks whatever --warmup says:
    # SETTLE_STEPS untimed steps come before the warm-up steps (reported as "settle_steps").
    # The same measurement is taken first with the caller's warm-up alone ("ms_per_step_unsettled"), so that a
    # change of the kernels and a change of the clocks cannot be mistaken for one another between runs.
    for i in range(args.warmup):
        sfa_step(i)
    torch.cuda.synchronize()
    evu0, evu1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    tu0 = time.perf_counter()
    evu0.record()
    for i in range(args.steps):
        sfa_step(i)
    evu1.record()
    torch.cuda.synchronize()
    ms_per_step_unsettled = (time.perf_counter() - tu0) / args.steps * 1e3
    ev_avg_ms_unsettled = evu0.elapsed_time(evu1) / args.steps
    for i in range(SETTLE_STEPS):
        sfa_step(i)
    for i in range(args.warmup):
        sfa_step(i)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for i in range(args.steps):
        sfa_step(i)
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    # Device-side duration of a step's launches: one pair of HIP events around the timed steps, on the stream
    # the kernels run on (the wall clock above also holds the first launch's latency and the final
    # synchronisation, which 20 steps do not amortise); the per-step minimum from a second pass with an
    # event pair around every step.
    ev_avg_ms = ev0.elapsed_time(ev1) / args.steps
    _, _, ev_min_ms = time_events(sfa_step, args.steps, 0, torch)

    cur_seqs = [min(L, K) for L in lengths]
    byt, flops = sfa_algorithmic_work(cur_seqs, NQ)
    # what the committed counter summaries must have been taken with to still describe this library
    from pypto_amd import _native
    C = _native.load()
    lib_version = C.version()
    ws_bytes = C.sfa_quant_workspace_bytes(B, S1, NQ, 1, K, 128, int(sfa_d.block_table.shape[1]), int(sfa_d.key_nope_2d.shape[0]),
                                           float(sfa.softmax_scale), 0)
    key_splits = max(ws_bytes // (B * S1 * NQ * (512 * 2 + 8)), 1)
    combine_ns = 2 if key_splits <= 2 else (4 if key_splits <= 4 else 8)      # splits the merge kernel holds in flight
    achieved_tflops = flops / (ev_avg_ms * 1e-3) / 1e12
    achieved_gbs = byt / (ev_avg_ms * 1e-3) / 1e9

    # ------------------------------------------------------------------ the same step over packed cache rows
    from pypto_amd.synthetic import pack_nope_cache
    packed = pack_nope_cache(sfa_d.key_nope_2d, sfa_d.key_rope_2d, sfa_d.k_nope_scales)
    out_p = torch.zeros_like(out)

    def packed_step(i):
        pypto_amd.sparse_attention_antiquant_d(sfa_d.query_nope, sfa_d.query_rope, packed, sel[i % ROT],
                                               sfa_d.block_table, sfa_d.kv_act_seqs, out_p, NQ, 1,
                                               sfa.softmax_scale, K, 128, sfa.max_blocknum_perbatch, None)
    # timed like the steps above, and after as many settling steps: packing the cache left the device idle
    packed_avg_ms = time_batch(packed_step, max(args.steps // 2, 5), SETTLE_STEPS, torch)
    sfa_step(0)
    packed_step(0)
    torch.cuda.synchronize()
    packed_same = bool(torch.equal(out.view(torch.int16), out_p.view(torch.int16)))
    del packed

    # ------------------------------------------------------------------ indexer timings
    res = torch.empty([B, 1, K], dtype=torch.int32, device=dev)

    def li_step(i):
        pypto_amd.lightning_indexer_decode(idx_queries[i % ROT], li_d.idx_query_scale, li_d.idx_key_cache,
                                           li_d.idx_key_scale, li_d.idx_weight, li_d.act_seq_key, li_d.block_table,
                                           res, None, None, K)
    li2_avg_ms = time_batch(li_step, max(args.steps // 2, 40), 20, torch)
    li2_bytes = indexer_algorithmic_bytes(lengths, 4)

    li1 = gen_indexer_inputs(4, 1, config_lengths(1), selected_count=K, seed=1, variant="fp32").to(dev)

    def li1_step(i):
        pypto_amd.lightning_indexer_decode(li1.idx_query, li1.idx_query_scale, li1.idx_key_cache, li1.idx_key_scale,
                                           li1.idx_weight, li1.act_seq_key, li1.block_table, li1.topk_res, None, None,
                                           K)
    li1_avg_ms = time_batch(li1_step, max(args.steps // 2, 40), 20, torch)
    li1_bytes = indexer_algorithmic_bytes(config_lengths(1), 4)
    del li1

    # configs[3]'s indexer: B=64, two query tokens per sequence (the pair shares one pass over the keys)
    len3 = config_lengths(3, seed=3)
    li3 = gen_indexer_inputs(64, 2, len3, selected_count=K, seed=3, variant="fp32").to(dev)

    def li3_step(i):
        pypto_amd.lightning_indexer_decode(li3.idx_query, li3.idx_query_scale, li3.idx_key_cache, li3.idx_key_scale,
                                           li3.idx_weight, li3.act_seq_key, li3.block_table, li3.topk_res, None, None,
                                           K)
    li3_avg_ms = time_batch(li3_step, max(args.steps // 4, 20), 10, torch)
    # per sequence: the keys once, two tokens' queries, factors and results
    li3_bytes = sum(L * (128 + 4) + 2 * (64 * 128 + 64 * 8 + K * 4) + 4 * math.ceil(L / 128) for L in len3)
    del li3

    # ------------------------------------------------------------------ indexer prolog (projection stage)
    # the side legs must not cost the headline line: a failure there is reported in its field
    def side_leg(fn):
        try:
            return fn(torch, dev, pypto_amd)
        except Exception as e:                                # noqa: BLE001 -- reported, not swallowed
            torch.cuda.synchronize()
            return {"error": f"{type(e).__name__}: {e}"}
    prolog = side_leg(prolog_leg)
    mla_prolog = side_leg(mla_prolog_leg)
    fused_prolog = side_leg(fused_prolog_leg)
    # ... and at the batch of the headline workload (32 sequences, one token each), fewer weight sets per graph
    for leg, fn, calls in ((prolog, prolog_leg, 20), (mla_prolog, mla_prolog_leg, 6), (fused_prolog, fused_prolog_leg, 6)):
        leg["batch_of_32"] = side_leg(lambda t_, d_, p_, fn=fn, calls=calls: fn(t_, d_, p_, b=B, s1=1, calls=calls))

    # ------------------------------------------------------------------ CPU baseline (bounded sample)
    cpu = None
    if not args.no_cpu_baseline:
        from oracle import c_oracle
        nthreads = min(c_oracle.get_threads(), os.cpu_count() or 1)
        c_oracle.set_threads(nthreads)
        # the whole batch, repeated until about ten seconds of host work have been timed
        idx_cpu = sel[0].cpu()
        reps, t_cpu = 0, 0.0
        while t_cpu < 10.0 and reps < 400:
            t_cpu0 = time.perf_counter()
            c_oracle.sfa_quant(sfa.query_nope, sfa.query_rope, sfa.key_nope_2d, sfa.key_rope_2d, sfa.k_nope_scales,
                               idx_cpu, sfa.block_table, sfa.kv_act_seqs, B, 1, NQ, K, 128, sfa.softmax_scale,
                               s2_tile=0)
            t_cpu += time.perf_counter() - t_cpu0
            reps += 1
        cpu = {"value": reps * B / t_cpu, "unit": "tokens/s", "cores": nthreads, "kind": "port",
               "sample": f"the same batch of {B} sequences, {reps} passes of the scalar C golden (OpenMP over "
                         f"heads), {t_cpu:.1f} s"}
        # configs[0] (B=1, 16 heads, top-k 256, the reference's own CPU-sized case) in the golden's literal form --
        # one Python iteration per selected key, as the reference gathers them
        # (deepseekv32_sparse_flash_attention_quant.py:215-228) -- and in the vectorised torch form of the same golden
        from oracle import sfa_oracle
        c0 = gen_sfa_inputs(1, 1, 16, config_lengths(0), topk=256, seed=0, shuffle_table=False)
        a0 = (c0.q_bsnd(), c0.key_nope_2d, c0.key_rope_2d, c0.k_nope_scales, c0.topk_indices, c0.block_table,
              c0.actual_seq, c0.block_size, c0.softmax_scale, c0.topk)
        forms = {}
        for name, fn in (("loop_form", sfa_oracle.sfa_literal_loops), ("vectorised", sfa_oracle.sfa_single_pass)):
            fn(*a0)
            n0, t0c = 0, 0.0
            while t0c < 1.0 and n0 < 2000:
                tc = time.perf_counter()
                fn(*a0)
                t0c += time.perf_counter() - tc
                n0 += 1
            forms[name] = {"tokens_per_s": n0 / t0c, "ms_per_call": t0c / n0 * 1e3, "calls": n0}
        cpu["configs[0]_torch_golden"] = {"workload": "configs[0]: B=1 S_q=1 16 heads topk=256 KV 4096", "torch_threads": torch.get_num_threads(), **forms}

    line = {
        "metric": "sfa_decode_tokens_per_s",
        "value": B * S1 / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_steps": SETTLE_STEPS,
        "ms_per_step": ms_per_step,
        "ms_per_step_unsettled": ms_per_step_unsettled,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "configs[2]: SFA decode B=32 S_q=1 128 heads d=576/512 topk=2048 (from the indexer) "
                               "int8 latent KV + 4 fp32 scales/token + bf16 rope, KV 8192-65536 paged bs=128, "
                               f"shuffled block table, {ROT} rotating selections",
                   "kv_rows": int(sfa.key_nope_2d.shape[0]), "sum_kv_len": int(sum(lengths))},
        "roofline": {"bound": "mfma", "achieved": achieved_tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved_tflops / PEAK_BF16_TFLOPS,
                     "traffic": measured_traffic(TRAFFIC_FILE, "traffic_bytes_per_step", lib_version,
                                                 {"key_splits": key_splits}),
                     "kernel": "sfa_decode_kernel<4>" + (f" + sfa_combine_kernel<{combine_ns}>" if key_splits > 1 else "") + " (one step)",
                     "key_splits": int(key_splits),
                     "launch_ms_avg": ev_avg_ms, "launch_ms_min": ev_min_ms, "launch_ms_avg_unsettled": ev_avg_ms_unsettled,
                     "frac_unsettled": flops / (ev_avg_ms_unsettled * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, "flops_per_launch": flops},
        "roofline_hbm": {"bound": "hbm", "achieved": achieved_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": achieved_gbs / PEAK_HBM_GBS, "bytes_per_launch": byt},
        "packed_cache": {"operator": "sparse_attention_antiquant_d", "us_per_step": packed_avg_ms * 1e3,
                         "bit_identical_to_three_array_result": packed_same},
        "indexer": {"configs[2]_us_per_step": li2_avg_ms * 1e3, "configs[2]_hbm_frac": li2_bytes / (li2_avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                    "configs[1]_us_per_step": li1_avg_ms * 1e3, "configs[1]_hbm_frac": li1_bytes / (li1_avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                    "bytes_configs[2]": li2_bytes, "bytes_configs[1]": li1_bytes,
                    "traffic_configs[2]": measured_traffic(LI_TRAFFIC_FILE, "indexer_traffic_bytes_configs2", lib_version),
                    "traffic_configs[1]": measured_traffic(LI_TRAFFIC_FILE, "indexer_traffic_bytes_configs1", lib_version),
                    "configs[3]_us_per_step": li3_avg_ms * 1e3,
                    "configs[3]_hbm_frac": li3_bytes / (li3_avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, "bytes_configs[3]": li3_bytes,
                    "scale_dtype": "fp32", "weight_dtype": "bf16"},
        "indexer_prolog": prolog,
        "mla_prolog": mla_prolog,
        "mla_indexer_prolog": fused_prolog,
        "cpu_baseline": cpu,
    }
    if args.other_shapes:
        line["other_shapes"] = other_shapes_leg(torch, pypto_amd, dev)
    if args.prefill_prologs:
        line["prefill_prologs"] = prefill_prologs_leg(torch, pypto_amd, dev)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
