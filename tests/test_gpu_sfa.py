"""Parity of the HIP sparse-flash-attention path (through the operator, pybind11 and the C ABI)
against the CPU oracle.  Tolerance: max-abs 2e-2 and mean-rel 5e-3 (mean|d| / mean|ref|) in bf16."""
import pytest
import torch

import pypto_amd
from pypto_amd import sparse_flash_attention_quant_impl as impl
from pypto_amd.synthetic import gen_sfa_inputs, config_lengths
from pypto_amd.utils import attention_error_stats

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_REL = 2e-2, 5e-3


def run_op(inp, num_splits=0, entry="d"):
    dev = torch.device("cuda:0")
    d = inp.to(dev)
    out = torch.full([inp.b, inp.s1, inp.n_q, 512], float("nan"), dtype=torch.bfloat16, device=dev)
    ts = [pypto_amd.from_torch(t, name=f"in{i}") for i, t in enumerate(d.operator_tensors())]
    if num_splits:
        impl._launch(*ts, pypto_amd.from_torch(out), inp.n_q, 1, inp.softmax_scale, inp.topk, inp.block_size,
                     inp.max_blocknum_perbatch, num_splits=num_splits)
    else:
        fn = pypto_amd.sparse_flash_attention_quant_d if entry == "d" else pypto_amd.sparse_flash_attention_quant_p
        cfg = pypto_amd.SaTileShapeConfig(128, 2048, [128] * 6, [8, 2048], [128] * 6, [64, 128])
        ret = fn(*ts, pypto_amd.from_torch(out, name="out"), inp.n_q, 1, inp.softmax_scale, inp.topk,
                 inp.block_size, inp.max_blocknum_perbatch, cfg)
        assert ret is None
    torch.cuda.synchronize()
    return out.cpu()


def oracle(inp, online_tile=None):
    from oracle import sfa_oracle as so
    args = (inp.q_bsnd(), inp.key_nope_2d, inp.key_rope_2d, inp.k_nope_scales, inp.topk_indices, inp.block_table,
            inp.actual_seq, inp.block_size, inp.softmax_scale, inp.topk)
    if online_tile:
        return so.sfa_online(*args, s2_tile=online_tile)
    return so.sfa_single_pass(*args)


def check(out, ref, what):
    assert not torch.isnan(out).any(), f"{what}: NaN in output"
    max_abs, mean_rel = attention_error_stats(out, ref)
    print(f"{what}: max_abs={max_abs:.4g} mean_rel={mean_rel:.4g}", flush=True)
    assert max_abs <= MAX_ABS and mean_rel <= MEAN_REL, (what, max_abs, mean_rel)


def test_config0_tiny_decode():
    """B=1, 16 heads, KV 4096 with an identity table, top-k 256."""
    inp = gen_sfa_inputs(1, 1, 16, config_lengths(0), topk=256, seed=0, shuffle_table=False)
    out = run_op(inp)
    check(out, oracle(inp), "cfg0 vs single-pass golden")
    check(out, oracle(inp, online_tile=32), "cfg0 vs online golden")
    # Accuracy against the exact (fp64) attention over the same de-quantised bf16 keys: the kernel is
    # held to the error the reference's own goldens make.  (The reference driver's comparator, rtol
    # 5e-3 with 0.5 % outliers, separates even the reference's two goldens from each other -- 17 % of
    # the elements of this case differ by more than that between them, one bf16 ulp being 0.4-0.8 % --
    # so it is reported here, not asserted.)
    from oracle import sfa_oracle as so
    kn = so.dequant_kn(inp.key_nope_2d, inp.k_nope_scales).double()
    k = torch.cat([kn, inp.key_rope_2d.double()], dim=-1)
    sel = inp.topk_indices[0].long()
    truth = torch.nn.functional.scaled_dot_product_attention(
        inp.q_bsnd()[0, 0].double()[None], k[sel][None], kn[sel][None], scale=inp.softmax_scale)[0].float()
    err_gpu = attention_error_stats(out[0, 0], truth)[1]
    err_gold = attention_error_stats(oracle(inp)[0, 0], truth)[1]
    print(f"mean-rel error vs fp64: kernel {err_gpu:.4g}, single-pass golden {err_gold:.4g}", flush=True)
    assert err_gpu <= 1.25 * err_gold + 1e-4
    ref = oracle(inp, online_tile=32).float()
    d = (out.float() - ref).abs()
    print(f"outliers under the reference comparator vs online golden: "
          f"{float((d > 1e-4 + 5e-3 * ref.abs()).float().mean()):.4f}", flush=True)


@pytest.mark.parametrize("n_q,b,s1,act,topk", [
    (128, 2, 1, [700, 333], 256),        # ragged, partial last tile
    (128, 3, 2, [65, 1, 4096], 128),     # two query tokens per sequence; act=1 gives an empty first row
    (64, 2, 1, [100, 31], 64),           # two-wave workgroups
    (16, 2, 2, [40, 2], 32),             # single-wave workgroups
    (1, 1, 1, [50], 64),                 # one head
    (200, 1, 1, [300], 96),              # two head groups, second one partial
    (128, 1, 4, [3], 64),                # s1 = 4 with act < s1: rows 0 have no keys
])
def test_ragged_shapes(n_q, b, s1, act, topk):
    inp = gen_sfa_inputs(b, s1, n_q, act, topk=topk, seed=n_q + b + s1)
    out = run_op(inp)
    ref = oracle(inp)
    check(out, ref, f"nq={n_q} b={b} s1={s1} act={act}")
    for bi in range(b):
        for si in range(s1):
            if act[bi] - s1 + 1 + si <= 0:
                assert torch.all(out[bi, si] == 0)


@pytest.mark.parametrize("splits", [2, 3, 4, 5, 8, 12])   # the combine kernel takes 2, 4 or 8 splits per trip
def test_key_splits_agree_with_single_workgroup(splits):
    inp = gen_sfa_inputs(2, 1, 128, [3000, 500], topk=1024, seed=21)
    base = run_op(inp, num_splits=1)
    check(base, oracle(inp), "unsplit")
    out = run_op(inp, num_splits=splits)
    check(out, oracle(inp), f"{splits} splits")
    max_abs, _ = attention_error_stats(out, base)
    assert max_abs <= 2 ** -6


@pytest.mark.parametrize("b", [20, 44])
def test_batches_that_do_not_divide_the_compute_units(b):
    """Batches whose rows do not spread evenly over the eight XCDs (20 rows: three on some, two on others; 44: six and
    five): the library's own split count (fewer, longer splits instead of a second, nearly empty round of
    workgroups) against the same launch with one workgroup per row, at the top-k of the benchmark."""
    inp = gen_sfa_inputs(b, 1, 128, [4096 - 61 * i for i in range(b)], topk=2048, seed=b)
    base = run_op(inp, num_splits=1)
    out = run_op(inp)
    max_abs, mean_rel = attention_error_stats(out, base)
    print(f"b={b}: default splits vs one workgroup per row: max_abs={max_abs:.4g} mean_rel={mean_rel:.4g}", flush=True)
    assert max_abs <= 2 ** -6
    check(out, oracle(inp), f"b={b}, default splits")


def test_prefill_entry_point_and_causal_rows():
    """Chunked-prefill shape in miniature: every query row t sees min(t+1, topk) keys."""
    inp = gen_sfa_inputs(1, 96, 128, [96], topk=64, seed=5)
    out = run_op(inp, entry="p")
    check(out, oracle(inp), "prefill s1=96")


def test_large_scores_jump_forces_rescale():
    """Keys ordered so the running maximum jumps by far more than the lazy-rescale threshold."""
    inp = gen_sfa_inputs(1, 1, 128, [512], topk=512, seed=9, shuffle_table=False)
    inp.topk_indices[0] = torch.arange(512, dtype=torch.int32)
    q = inp.q_bsnd()[0, 0].float()                       # [128, 576]
    # make the last 64 keys strongly aligned with the mean query direction of the nope part
    inp.query_nope[:] = (inp.query_nope.float() * 0.2 + 3.0).to(torch.bfloat16)
    inp.key_nope_2d[448:] = 127
    inp.k_nope_scales[448:] = 0.02
    out = run_op(inp, num_splits=1)
    check(out, oracle(inp), "late large keys")
    out = run_op(inp, num_splits=4)
    check(out, oracle(inp), "late large keys, 4 splits")


def test_identical_keys_invariant_full_width():
    inp = gen_sfa_inputs(2, 1, 128, [5000, 9000], topk=2048, seed=3)
    inp.topk_indices[:] = 1234
    out = run_op(inp)
    from oracle import sfa_oracle as so
    for bi in range(2):
        phys = int(so.page_translate(torch.tensor([1234]), inp.block_table[bi], 128)[0])
        v = so.dequant_kn(inp.key_nope_2d[phys:phys + 1], inp.k_nope_scales[phys:phys + 1]).float()
        # softmax over identical scores is uniform; P = bf16(1) and the row sum 2048 are exact
        assert torch.equal(out[bi, 0].float(), v.expand(128, -1))


# ------------------------------------------------------------------ packed 656-byte cache rows

def run_packed(inp, entry="d"):
    from pypto_amd.synthetic import pack_nope_cache
    dev = torch.device("cuda:0")
    d = inp.to(dev)
    packed = pack_nope_cache(d.key_nope_2d, d.key_rope_2d, d.k_nope_scales)
    out = torch.full([inp.b, inp.s1, inp.n_q, 512], float("nan"), dtype=torch.bfloat16, device=dev)
    fn = pypto_amd.sparse_attention_antiquant_d if entry == "d" else pypto_amd.sparse_attention_antiquant_p
    cfg = pypto_amd.SaTileShapeConfig(128, 2048, [128] * 6, [8, 2048], [128] * 6, [64, 128])
    ret = fn(pypto_amd.from_torch(d.query_nope), pypto_amd.from_torch(d.query_rope), pypto_amd.from_torch(packed),
             pypto_amd.from_torch(d.topk_indices), pypto_amd.from_torch(d.block_table), pypto_amd.from_torch(d.kv_act_seqs),
             pypto_amd.from_torch(out, name="out"), inp.n_q, 1, inp.softmax_scale, inp.topk, inp.block_size,
             inp.max_blocknum_perbatch, cfg)
    assert ret is None
    torch.cuda.synchronize()
    return out.cpu(), packed.cpu()


@pytest.mark.parametrize("n_q,b,s1,act,topk,entry", [
    (128, 2, 1, [5000, 3000], 2048, "d"),      # decode, key splits
    (16, 1, 1, [4096], 256, "d"),              # the tiny configuration
    (128, 1, 3, [700], 512, "p"),              # prefill entry, causal rows
    (40, 3, 2, [300, 1, 64], 128, "d"),        # head count that fills no wave, rows without keys
])
def test_packed_cache_operator(n_q, b, s1, act, topk, entry):
    """sparse_attention_antiquant over packed rows: against its golden, and bit-identical to the
    three-array operator on the same data (same kernel, other row pitches)."""
    from oracle import sfa_oracle as so
    inp = gen_sfa_inputs(b, s1, n_q, act, topk=topk, seed=17 + n_q)
    out, packed = run_packed(inp, entry)
    ref = so.sa_antiquant_single_pass(inp.q_bsnd(), packed, inp.topk_indices, inp.block_table, inp.actual_seq,
                                      inp.block_size, inp.softmax_scale, inp.topk)
    check(out, ref, f"packed nq={n_q} b={b} s1={s1} act={act} topk={topk}")
    assert torch.equal(out.view(torch.int16), run_op(inp, entry=entry).view(torch.int16))


# ------------------------------------------------------------------ non-quantized (bf16) latent cache

@pytest.mark.parametrize("n_q,b,s1,act,topk", [
    (128, 2, 1, [5000, 3000], 2048),
    (16, 1, 1, [4096], 256),
    (64, 2, 2, [300, 70], 128),
])
def test_bf16_latent_cache_branch(n_q, b, s1, act, topk):
    """key_nope_2d in bf16, no scales: against the golden's non-quantized branch, and -- fed with exactly
    the values the int8 cache de-quantises to -- bit-identical to the quantized operator."""
    from oracle import sfa_oracle as so
    inp = gen_sfa_inputs(b, s1, n_q, act, topk=topk, seed=23 + n_q)
    kn_bf16 = so.dequant_kn(inp.key_nope_2d, inp.k_nope_scales)
    assert kn_bf16.dtype == torch.bfloat16
    dev = torch.device("cuda:0")
    d = inp.to(dev)
    out = torch.full([inp.b, inp.s1, inp.n_q, 512], float("nan"), dtype=torch.bfloat16, device=dev)
    ret = pypto_amd.sparse_flash_attention_quant_d(d.query_nope, d.query_rope, kn_bf16.to(dev), d.key_rope_2d, None,
                                                   d.topk_indices, d.block_table, d.kv_act_seqs, out, inp.n_q, 1,
                                                   inp.softmax_scale, inp.topk, inp.block_size,
                                                   inp.max_blocknum_perbatch, None)
    assert ret is None
    torch.cuda.synchronize()
    out = out.cpu()
    ref = so.sfa_single_pass(inp.q_bsnd(), kn_bf16, inp.key_rope_2d, None, inp.topk_indices, inp.block_table,
                             inp.actual_seq, inp.block_size, inp.softmax_scale, inp.topk, is_kn_quant=False)
    check(out, ref, f"bf16 cache nq={n_q} b={b} s1={s1}")
    assert torch.equal(out.view(torch.int16), run_op(inp).view(torch.int16))


@pytest.mark.parametrize("scale", [-0.0416666679084301, 0.0, 0.25])
def test_softmax_scale_of_any_sign(scale):
    """The kernel scales scores inside the exponent and wants a positive factor: a negative one moves its
    sign into the query, a zero one gives uniform weights.  All three against the golden, with key splits."""
    inp = gen_sfa_inputs(2, 1, 128, [3000, 200], topk=512, seed=41)
    inp.softmax_scale = scale
    ref = oracle(inp)
    check(run_op(inp), ref, f"scale={scale}")
    check(run_op(inp, num_splits=4), ref, f"scale={scale}, 4 splits")
