"""Pins the sparse-flash-attention oracle (oracle/sfa_oracle.py, oracle/oracle_c.c).

Every check here is independent of the oracle's own formulae: a known answer from
the reference's documentation, an exhaustive bit-level rounding, a library
routine (fp64 scaled_dot_product_attention) on the dense special case, invariants
of the mathematics, or the second, independently written C statement.
"""
import math
import struct

import numpy as np
import pytest
import torch

from oracle import sfa_oracle as so
from pypto_amd.synthetic import gen_sfa_inputs, gen_block_table
from pypto_amd.utils import attention_error_stats


# ---------------------------------------------------------------- paging / gather

def test_gather_known_answer_from_reference_docstring():
    # python/pypto/experimental.py:64-87 of the reference
    param = torch.tensor([[10 * r + c for c in range(4)] for r in range(6)], dtype=torch.float16)
    out = so.gather_rows(param, torch.tensor([[0, 4, 3]], dtype=torch.int32),
                         torch.tensor([[0, 2, 1]], dtype=torch.int32), 2)
    assert out.tolist() == [[0, 1, 2, 3], [20, 21, 22, 23], [50, 51, 52, 53]]


@pytest.mark.parametrize("seed", [42, 123])
def test_gather_row_col_recipe(seed):
    # python/tests/st/test_gatherinub.py:89-155 of the reference: buffer value 10*row+col
    g = torch.Generator().manual_seed(seed)
    bs, nblk, hidden, k = 16, 12, 8, 40
    param = (10 * torch.arange(nblk * bs).reshape(-1, 1) + torch.arange(hidden).reshape(1, -1)).to(torch.float32)
    table = torch.randperm(nblk, generator=g).to(torch.int32)
    idx = torch.randint(0, nblk * bs, [k], generator=g, dtype=torch.int32)
    out = so.gather_rows(param, idx, table, bs)
    for j in range(k):
        li = int(idx[j])
        phys = int(table[li // bs]) * bs + li % bs      # plain-python page walk
        assert out[j].tolist() == [10 * phys + c for c in range(hidden)]


# ---------------------------------------------------------------- de-quantisation

def _bf16_bits_rne(f32_value: np.float32) -> int:
    """fp32 -> bf16 bits, round half to even, written with Python integers only."""
    u = struct.unpack("<I", struct.pack("<f", float(f32_value)))[0]
    hi, lo = u >> 16, u & 0xFFFF
    if lo > 0x8000 or (lo == 0x8000 and (hi & 1)):
        hi += 1
    return hi & 0xFFFF


def test_dequant_exhaustive_all_int8(c_oracle):
    scales = torch.tensor([0.005, 0.0123456, 0.02, 1.0, 3.1415927e-3, 7.7e-5, 0.3333333, 1e-8],
                          dtype=torch.float32)
    vals = torch.arange(-128, 128, dtype=torch.int8)
    for s in scales:
        rows = vals.reshape(1, 256).repeat(1, 2)                      # [1, 512]
        sc = s.reshape(1, 1).repeat(1, 4)
        got = so.dequant_kn(rows, sc).view(torch.int16).reshape(-1)[:256]
        for i, v in enumerate(range(-128, 128)):
            prod = np.float32(v) * np.float32(s.item())               # the fp32 multiply
            want = _bf16_bits_rne(prod)
            assert (int(got[i]) & 0xFFFF) == want, (v, float(s))
            assert c_oracle.lib().oracle_f32_to_bf16(float(prod)) == want


def test_dequant_uses_scale_of_its_128_channel_group():
    rows = torch.ones([3, 512], dtype=torch.int8)
    sc = torch.tensor([[1.0, 2.0, 4.0, 8.0]] * 3, dtype=torch.float32)
    out = so.dequant_kn(rows, sc).to(torch.float32)
    for g, v in enumerate([1.0, 2.0, 4.0, 8.0]):
        assert torch.all(out[:, 128 * g:128 * (g + 1)] == v)


# ---------------------------------------------------------------- attention core

def _dense_case(seed, n_q=8, length=256, b=1):
    inp = gen_sfa_inputs(b, 1, n_q, [length] * b, topk=length, seed=seed, shuffle_table=False)
    return inp


def _oracle(inp, fn=so.sfa_single_pass, **kw):
    return fn(inp.q_bsnd(), inp.key_nope_2d, inp.key_rope_2d, inp.k_nope_scales, inp.topk_indices,
              inp.block_table, inp.actual_seq, inp.block_size, inp.softmax_scale, inp.topk, **kw)


def test_dense_special_case_matches_fp64_sdpa():
    """topk == L with an identity table is textbook softmax(QK^T s)V."""
    inp = _dense_case(1)
    out = _oracle(inp)
    kn = so.dequant_kn(inp.key_nope_2d, inp.k_nope_scales).to(torch.float64)
    k = torch.cat([kn, inp.key_rope_2d.to(torch.float64)], dim=-1)
    q = inp.q_bsnd()[0, 0].to(torch.float64)
    ref = torch.nn.functional.scaled_dot_product_attention(q[None], k[None], kn[None], scale=inp.softmax_scale)[0]
    max_abs, mean_rel = attention_error_stats(out[0, 0], ref.to(torch.float32))
    assert max_abs <= 2e-2 and mean_rel <= 5e-3, (max_abs, mean_rel)
    # the check has teeth: dropping the rope columns, or the softmax scale, is far outside it
    ref_norope = torch.nn.functional.scaled_dot_product_attention(
        q[None, :, :512], kn[None], kn[None], scale=inp.softmax_scale)[0]
    assert attention_error_stats(out[0, 0], ref_norope.to(torch.float32))[1] > 5e-2
    ref_noscale = torch.nn.functional.scaled_dot_product_attention(q[None], k[None], kn[None], scale=1.0)[0]
    assert attention_error_stats(out[0, 0], ref_noscale.to(torch.float32))[1] > 5e-2


def test_identical_keys_give_that_value_row():
    inp = _dense_case(2, n_q=4, length=128)
    inp.topk_indices[:] = 77
    out = _oracle(inp)
    v = so.dequant_kn(inp.key_nope_2d[77:78], inp.k_nope_scales[77:78]).to(torch.float32)
    # uniform softmax over identical rows: p = 1/128 exactly, sum of 128 equal fp32 terms is exact
    assert torch.equal(out[0, 0].to(torch.float32), v.expand(4, -1))


def test_permuting_selected_indices_changes_nothing_material():
    inp = gen_sfa_inputs(1, 1, 8, [1024], topk=256, seed=3)
    a = _oracle(inp)
    g = torch.Generator().manual_seed(9)
    inp.topk_indices[0] = inp.topk_indices[0][torch.randperm(256, generator=g)]
    b = _oracle(inp)
    assert attention_error_stats(a, b)[0] <= 2 ** -6    # fp32 summation order only: at most a bf16 ulp


def test_page_table_invariance():
    """Physically shuffling blocks and recording it in the table leaves the result bit-identical."""
    ident = gen_sfa_inputs(2, 1, 4, [700, 300], topk=128, seed=4, shuffle_table=False)
    out_a = _oracle(ident)
    g = torch.Generator().manual_seed(5)
    perm = torch.randperm(ident.block_num, generator=g)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(ident.block_num)
    bs = ident.block_size

    def move(x):
        return x.reshape(ident.block_num, bs, -1)[inv].reshape(ident.block_num * bs, -1).contiguous()
    shuf = gen_sfa_inputs(2, 1, 4, [700, 300], topk=128, seed=4, shuffle_table=False)
    shuf.key_nope_2d, shuf.key_rope_2d, shuf.k_nope_scales = move(ident.key_nope_2d), move(ident.key_rope_2d), \
        move(ident.k_nope_scales)
    tbl = ident.block_table.clone()
    valid = tbl >= 0
    tbl[valid] = perm[tbl[valid].long()].to(torch.int32)
    shuf.block_table = tbl
    assert torch.equal(out_a, _oracle(shuf))


@pytest.mark.parametrize("act,s1,topk,expect", [
    (1, 2, 8, [0, 1]), (2, 2, 8, [1, 2]), (0, 1, 8, [0]), (8, 1, 8, [8]), (9, 1, 8, [8]), (9, 2, 8, [8, 8]),
    (8, 2, 8, [7, 8]), (2047, 1, 2048, [2047]), (2049, 1, 2048, [2048]), (3, 4, 8, [0, 1, 2, 3]),
])
def test_cur_seq_formula(act, s1, topk, expect):
    assert [so.cur_seq_of(act, s1, s, topk) for s in range(s1)] == expect


def test_rows_without_keys_are_zero_and_only_first_cur_seq_entries_matter():
    inp = gen_sfa_inputs(2, 2, 4, [1, 300], topk=64, seed=6)
    out = _oracle(inp)
    assert torch.all(out[0, 0] == 0)          # act=1, s1=2: first token has no key
    assert torch.any(out[0, 1] != 0)
    # entries past cur_seq are ignored, whatever they hold
    inp2 = gen_sfa_inputs(2, 2, 4, [1, 300], topk=64, seed=6)
    inp2.topk_indices[1, 1:] = 0
    inp2.topk_indices[0, :] = 0
    assert torch.equal(out, _oracle(inp2))


def test_causal_second_token_sees_one_more_key():
    inp = gen_sfa_inputs(1, 2, 2, [40], topk=64, seed=7)
    # token 0 attends 39 keys, token 1 attends 40
    assert int((inp.topk_indices[0] >= 0).sum()) == 39 and int((inp.topk_indices[1] >= 0).sum()) == 40


@pytest.mark.parametrize("tile", [32, 100, 256])
def test_online_softmax_agrees_with_single_pass(tile):
    inp = gen_sfa_inputs(2, 1, 8, [900, 200], topk=256, seed=8)
    a = _oracle(inp)
    b = _oracle(inp, fn=so.sfa_online, s2_tile=tile)
    max_abs, mean_rel = attention_error_stats(b, a)
    assert max_abs <= 2 ** -5 and mean_rel <= 4e-3, (max_abs, mean_rel)   # bf16 ulp noise only


def test_literal_loop_form_is_bit_identical_to_vectorised():
    inp = gen_sfa_inputs(2, 2, 4, [70, 33], topk=32, seed=10)
    args = (inp.q_bsnd(), inp.key_nope_2d, inp.key_rope_2d, inp.k_nope_scales, inp.topk_indices, inp.block_table,
            inp.actual_seq, inp.block_size, inp.softmax_scale, inp.topk)
    assert torch.equal(so.sfa_single_pass(*args), so.sfa_literal_loops(*args))


@pytest.mark.parametrize("tile", [0, 64])
def test_c_statement_agrees_with_torch_statement(c_oracle, tile):
    inp = gen_sfa_inputs(3, 2, 8, [513, 40, 1], topk=128, seed=11)
    if tile == 0:
        ref = _oracle(inp)
    else:
        ref = _oracle(inp, fn=so.sfa_online, s2_tile=tile)
    got = c_oracle.sfa_quant(inp.query_nope, inp.query_rope, inp.key_nope_2d, inp.key_rope_2d, inp.k_nope_scales,
                             inp.topk_indices, inp.block_table, inp.kv_act_seqs, inp.b, inp.s1, inp.n_q, inp.topk,
                             inp.block_size, inp.softmax_scale, s2_tile=tile)
    # same rounding points, different summation order and libm exp: a stray bf16 ulp at most
    d = (got.to(torch.float32) - ref.to(torch.float32)).abs()
    ulp = torch.maximum(ref.to(torch.float32).abs(), torch.tensor(2.0 ** -10)) * 2.0 ** -7
    assert float((d > ulp).float().mean()) == 0.0
    assert float((d > 0).float().mean()) < 0.02
    assert torch.all(got[2, 0] == 0)


# ------------------------------------------------------------------ packed 656-byte cache rows

def test_packed_row_byte_layout_known_answer():
    """A row written byte by byte with struct: 512 int8 | 64 bf16 (little endian) | 4 fp32 (little endian),
    the layout of the reference driver (deepseekv32_sparse_attention_antiquant.py:258-268)."""
    import struct
    from oracle import sfa_oracle as so
    ints = [((7 * i) % 256) - 128 for i in range(512)]
    bf16_bits = [0x3F80, 0xC000, 0x0000, 0x8000, 0x7F7F, 0x0001] + [0x3C00 + i for i in range(58)]   # 1.0, -2.0, +0, -0, max, tiny ...
    scales = [0.0078125, 1e-8, 3.5, 127.0]
    row = struct.pack("<512b", *ints) + struct.pack("<64H", *bf16_bits) + struct.pack("<4f", *scales)
    assert len(row) == 656
    cache = torch.frombuffer(bytearray(row + bytes(656)), dtype=torch.int8).reshape(2, 656)
    kn, kr, sc = so.unpack_nope_cache(cache)
    assert kn.dtype == torch.int8 and kn[0].tolist() == ints
    assert kr.dtype == torch.bfloat16 and kr[0].view(torch.int16).tolist() == [b - 65536 if b >= 32768 else b for b in bf16_bits]
    assert float(kr[0, 0]) == 1.0 and float(kr[0, 1]) == -2.0
    assert sc.dtype == torch.float32 and sc[0].tolist() == [struct.unpack("<f", struct.pack("<f", x))[0] for x in scales]
    assert kn[1].abs().sum() == 0 and sc[1].abs().sum() == 0


def test_packed_cache_round_trip_and_golden_equivalence():
    """pack (generator side) then unpack (oracle side) is the identity, and the packed golden equals the
    three-array golden on the same data."""
    from oracle import sfa_oracle as so
    from pypto_amd.synthetic import gen_sfa_inputs, pack_nope_cache
    inp = gen_sfa_inputs(2, 2, 8, [300, 70], topk=64, seed=5)
    packed = pack_nope_cache(inp.key_nope_2d, inp.key_rope_2d, inp.k_nope_scales)
    assert packed.shape == (inp.key_nope_2d.shape[0], 656) and packed.dtype == torch.int8
    kn, kr, sc = so.unpack_nope_cache(packed)
    assert torch.equal(kn, inp.key_nope_2d)
    assert torch.equal(kr.view(torch.int16), inp.key_rope_2d.view(torch.int16))
    assert torch.equal(sc.view(torch.int32), inp.k_nope_scales.view(torch.int32))
    a = so.sa_antiquant_single_pass(inp.q_bsnd(), packed, inp.topk_indices, inp.block_table, inp.actual_seq,
                                    inp.block_size, inp.softmax_scale, inp.topk)
    b = so.sfa_single_pass(inp.q_bsnd(), inp.key_nope_2d, inp.key_rope_2d, inp.k_nope_scales, inp.topk_indices,
                           inp.block_table, inp.actual_seq, inp.block_size, inp.softmax_scale, inp.topk)
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
