"""Seeded synthetic inputs for the sparse-attention path.

Host-side counterparts of the reference drivers' generators (paths relative to
the reference tree):

* ``gen_block_table``   examples/models/deepseek_v32_exp/
  deepseekv32_sparse_flash_attention_quant.py:257-295 and
  deepseekv32_lightning_indexer_quant.py:83-116 (random permutation of the
  physical blocks, ``-1`` in unused table slots)
* ``gen_sfa_inputs``    ...sparse_flash_attention_quant.py:298-388 (tensor names,
  shapes and layouts of the operator inputs; index rows are a random subset of
  the valid positions, or ``arange`` when fewer than ``topk`` exist)
* ``gen_indexer_inputs`` ...lightning_indexer_quant.py:119-181
* ``gen_indexer_prolog_inputs`` ...deepseekv32_lightning_indexer_prolog_quant.py:100-153
  (value ranges, tensor names and shapes; ``cache_index`` names the last ``s1``
  positions of every sequence, :76-84)
* ``gen_mla_prolog_inputs`` ...deepseekv32_mla_prolog_quant.py:329-453 for ``is_quant = (False, True)``
  (bf16 down-projections, per-channel int8 ``w_uqqr`` with its fp32 scales, value ranges)

Unlike the reference (global ``torch.manual_seed`` plus an unseeded
``np.random.permutation``) every generator here draws from an explicit
``torch.Generator`` so that a seed fully determines the inputs.

Value distributions follow the benchmark configurations: q ~ N(0,1) bf16, latent
KV int8 uniform in [-127,127] with fp32 scales uniform in [0.005,0.02] (four per
token), rope K ~ N(0,1) bf16; indexer q/k int8 uniform in [-127,127], per-token
scales, per-head weights N(0,1)/8.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import torch

BLOCK_SIZE = 128
KV_LORA_RANK = 512
ROPE_DIM = 64
IDX_HEADS = 64
IDX_DIM = 128


def gen_block_table(act_seq: Sequence[int], block_size: int, generator: Optional[torch.Generator] = None,
                    shuffle: bool = True, max_kv: Optional[int] = None):
    """Returns (block_num, block_table [B, ceil(max_kv/bs)] int32 with -1 padding)."""
    act = [int(a) for a in act_seq]
    per = [math.ceil(a / block_size) for a in act]
    block_num = sum(per)
    mb = math.ceil((max_kv if max_kv is not None else max(act + [1])) / block_size)
    mb = max(mb, 1)
    if shuffle:
        ids = torch.randperm(block_num, generator=generator).to(torch.int32)
    else:
        ids = torch.arange(block_num, dtype=torch.int32)
    table = -torch.ones([len(act), mb], dtype=torch.int32)
    pos = 0
    for i, n in enumerate(per):
        table[i, :n] = ids[pos:pos + n]
        pos += n
    return block_num, table


def gen_topk_indices(act_seq: Sequence[int], s1: int, topk: int, generator: torch.Generator,
                     causal: bool = True) -> torch.Tensor:
    """[B*S1, topk] int32.  Row (b, s) holds ``cur = min(max(act-S1+1+s,0), topk)`` valid
    entries: a random subset of the positions ``0 .. act-S1+s`` when more than
    ``topk`` exist, else ``arange``; the remainder is -1 (what the indexer pads with)."""
    b = len(act_seq)
    out = -torch.ones([b * s1, topk], dtype=torch.int32)
    for bi, act in enumerate(act_seq):
        for s in range(s1):
            eff = int(act) - (s1 - 1 - s) if causal else int(act)
            eff = max(eff, 0)
            if eff <= topk:
                out[bi * s1 + s, :eff] = torch.arange(eff, dtype=torch.int32)
            else:
                out[bi * s1 + s] = torch.randperm(eff, generator=generator)[:topk].to(torch.int32)
    return out


@dataclass
class SfaInputs:
    b: int
    s1: int
    n_q: int
    n_kv: int
    topk: int
    block_size: int
    block_num: int
    max_blocknum_perbatch: int
    softmax_scale: float
    actual_seq: List[int]
    query_nope: torch.Tensor      # [B*S1*Nq, 512] bf16
    query_rope: torch.Tensor      # [B*S1*Nq, 64]  bf16
    key_nope_2d: torch.Tensor     # [NB*bs, 512]   int8
    key_rope_2d: torch.Tensor     # [NB*bs, 64]    bf16
    k_nope_scales: torch.Tensor   # [NB*bs, 4]     fp32
    topk_indices: torch.Tensor    # [B*S1, topk]   int32
    block_table: torch.Tensor     # [B, MB]        int32
    kv_act_seqs: torch.Tensor     # [B]            int32

    def q_bsnd(self) -> torch.Tensor:
        """[B,S1,Nq,576] view (nope ‖ rope) as the goldens take it."""
        q = torch.cat([self.query_nope, self.query_rope], dim=-1)
        return q.reshape(self.b, self.s1, self.n_q, -1)

    def operator_tensors(self):
        return (self.query_nope, self.query_rope, self.key_nope_2d, self.key_rope_2d, self.k_nope_scales,
                self.topk_indices, self.block_table, self.kv_act_seqs)

    def to(self, device) -> "SfaInputs":
        kw = dict(self.__dict__)
        for k, v in kw.items():
            if isinstance(v, torch.Tensor):
                kw[k] = v.to(device)
        return SfaInputs(**kw)


def pack_nope_cache(key_nope_2d: torch.Tensor, key_rope_2d: torch.Tensor, k_nope_scales: torch.Tensor) -> torch.Tensor:
    """The packed cache of the antiquant operator: ``[rows, 656] int8`` = 512 int8 latent values |
    the 64 bf16 rope values as bytes | the 4 fp32 scales as bytes (the packing of the reference
    driver, deepseekv32_sparse_attention_antiquant.py:258-268)."""
    rows = key_nope_2d.shape[0]
    out = torch.zeros([rows, 656], dtype=torch.int8, device=key_nope_2d.device)
    out[:, :512] = key_nope_2d
    out[:, 512:640] = key_rope_2d.contiguous().view(torch.int8).reshape(rows, 128)
    out[:, 640:] = k_nope_scales.contiguous().view(torch.int8).reshape(rows, 16)
    return out


def gen_sfa_inputs(b: int, s1: int, n_q: int, actual_seq: Sequence[int], topk: int = 2048, seed: int = 0,
                   block_size: int = BLOCK_SIZE, shuffle_table: bool = True,
                   topk_indices: Optional[torch.Tensor] = None, block_table: Optional[torch.Tensor] = None,
                   block_num: Optional[int] = None) -> SfaInputs:
    g = torch.Generator().manual_seed(seed)
    act = [int(a) for a in actual_seq]
    assert len(act) == b
    if block_table is None:
        block_num, block_table = gen_block_table(act, block_size, g, shuffle=shuffle_table)
    rows = block_num * block_size
    t = b * s1
    q_nope = torch.randn([t * n_q, KV_LORA_RANK], generator=g).to(torch.bfloat16)
    q_rope = torch.randn([t * n_q, ROPE_DIM], generator=g).to(torch.bfloat16)
    kn = torch.randint(-127, 128, [rows, KV_LORA_RANK], generator=g, dtype=torch.int8)
    kr = torch.randn([rows, ROPE_DIM], generator=g).to(torch.bfloat16)
    scales = 0.005 + 0.015 * torch.rand([rows, 4], generator=g, dtype=torch.float32)
    if topk_indices is None:
        topk_indices = gen_topk_indices(act, s1, topk, g)
    d = KV_LORA_RANK + ROPE_DIM
    return SfaInputs(b=b, s1=s1, n_q=n_q, n_kv=1, topk=topk, block_size=block_size, block_num=block_num,
                     max_blocknum_perbatch=block_table.shape[1], softmax_scale=d ** -0.5, actual_seq=act,
                     query_nope=q_nope, query_rope=q_rope, key_nope_2d=kn, key_rope_2d=kr, k_nope_scales=scales,
                     topk_indices=topk_indices.reshape(t, topk).contiguous(), block_table=block_table,
                     kv_act_seqs=torch.tensor(act, dtype=torch.int32))


@dataclass
class IndexerInputs:
    b: int
    s1: int
    selected_count: int
    block_size: int
    block_num: int
    act_seq: List[int]
    idx_query: torch.Tensor        # [T, 64, 128]       int8
    idx_query_scale: torch.Tensor  # [T, 64]            fp16 | fp32
    idx_key_cache: torch.Tensor    # [NB, bs, 1, 128]   int8
    idx_key_scale: torch.Tensor    # [NB, bs, 1]        fp16 | fp32
    idx_weight: torch.Tensor       # [T, 64]            fp16 | bf16
    act_seq_key: torch.Tensor      # [B]                int32
    block_table: torch.Tensor      # [B, MB]            int32
    topk_res: torch.Tensor = field(default=None)  # [T, 1, k] int32 output buffer

    def operator_tensors(self):
        return (self.idx_query, self.idx_query_scale, self.idx_key_cache, self.idx_key_scale, self.idx_weight,
                self.act_seq_key, self.block_table, self.topk_res)

    def to(self, device) -> "IndexerInputs":
        kw = dict(self.__dict__)
        for k, v in kw.items():
            if isinstance(v, torch.Tensor):
                kw[k] = v.to(device)
        return IndexerInputs(**kw)


def gen_indexer_inputs(b: int, s1: int, act_seq: Sequence[int], selected_count: int = 2048, seed: int = 0,
                       variant: str = "fp16", block_size: int = BLOCK_SIZE, shuffle_table: bool = True,
                       block_table: Optional[torch.Tensor] = None, block_num: Optional[int] = None,
                       n_heads: int = IDX_HEADS, head_dim: int = IDX_DIM) -> IndexerInputs:
    """``variant='fp16'``: fp16 scales and weights (the reference's dtypes);
    ``variant='fp32'``: fp32 scales and bf16 weights (the benchmark configuration)."""
    g = torch.Generator().manual_seed(seed)
    act = [int(a) for a in act_seq]
    if block_table is None:
        block_num, block_table = gen_block_table(act, block_size, g, shuffle=shuffle_table)
    t = b * s1
    q = torch.randint(-127, 128, [t, n_heads, head_dim], generator=g, dtype=torch.int8)
    k = torch.randint(-127, 128, [block_num, block_size, 1, head_dim], generator=g, dtype=torch.int8)
    qs = 0.005 + 0.015 * torch.rand([t, n_heads], generator=g, dtype=torch.float32)
    ks = 0.005 + 0.015 * torch.rand([block_num, block_size, 1], generator=g, dtype=torch.float32)
    w = torch.randn([t, n_heads], generator=g, dtype=torch.float32) / 8
    if variant == "fp16":
        qs, ks, w = qs.to(torch.float16), ks.to(torch.float16), w.to(torch.float16)
    elif variant == "fp32":
        w = w.to(torch.bfloat16)
    else:
        raise ValueError(f"unknown variant {variant!r}")
    return IndexerInputs(b=b, s1=s1, selected_count=selected_count, block_size=block_size, block_num=block_num,
                         act_seq=act, idx_query=q, idx_query_scale=qs, idx_key_cache=k, idx_key_scale=ks,
                         idx_weight=w, act_seq_key=torch.tensor(act, dtype=torch.int32), block_table=block_table,
                         topk_res=torch.zeros([t, 1, selected_count], dtype=torch.int32))


@dataclass
class IndexerPrologInputs:
    b: int
    s1: int
    block_size: int
    block_num: int
    act_seq: List[int]
    x: torch.Tensor              # [T, h]                 bf16
    q_norm: torch.Tensor         # [T, q_lora_rank]       int8
    q_norm_scale: torch.Tensor   # [T, 1]                 fp32
    w_qb: torch.Tensor           # [q_lora_rank, N*128]   int8
    w_qb_scale: torch.Tensor     # [N*128, 1]             fp32
    wk: torch.Tensor             # [h, 128]               bf16
    w_proj: torch.Tensor         # [h, N]                 bf16
    ln_gamma_k: torch.Tensor     # [128]                  bf16
    ln_beta_k: torch.Tensor      # [128]                  bf16
    cos_idx_rope: torch.Tensor   # [T, 64]                bf16
    sin_idx_rope: torch.Tensor   # [T, 64]                bf16
    hadamard_q: torch.Tensor     # [128, 128]             bf16
    hadamard_k: torch.Tensor     # [128, 128]             bf16
    k_cache: torch.Tensor        # [NB, bs, 1, 128]       int8   (updated in place)
    k_cache_scale: torch.Tensor  # [NB, bs, 1, 1]         fp16   (updated in place)
    k_cache_index: torch.Tensor  # [T]                    int64
    block_table: torch.Tensor    # [B, MB]                int32

    def input_tensors(self):
        return (self.x, self.q_norm, self.q_norm_scale, self.w_qb, self.w_qb_scale, self.wk, self.w_proj,
                self.ln_gamma_k, self.ln_beta_k, self.cos_idx_rope, self.sin_idx_rope, self.hadamard_q,
                self.hadamard_k, self.k_cache, self.k_cache_scale, self.k_cache_index)

    def to(self, device) -> "IndexerPrologInputs":
        kw = dict(self.__dict__)
        for k, v in kw.items():
            if isinstance(v, torch.Tensor):
                kw[k] = v.to(device)
        return IndexerPrologInputs(**kw)


def gen_indexer_prolog_inputs(b: int, s1: int, act_seq: Sequence[int], seed: int = 0, h: int = 7168,
                              q_lora_rank: int = 1536, n_heads: int = IDX_HEADS, head_dim: int = IDX_DIM,
                              rope_dim: int = ROPE_DIM, block_size: int = BLOCK_SIZE,
                              affine_ln: bool = False) -> IndexerPrologInputs:
    """Value ranges of the reference generator: x, weights and Hadamard matrices uniform in (-1, 1) bf16,
    int8 operands uniform over the full range, scales uniform in (-1, 1), cos/sin of uniform angles, cache
    filled with random rows.  ``affine_ln`` draws gamma/beta at random instead of the reference's 1/0."""
    g = torch.Generator().manual_seed(seed)
    act = [int(a) for a in act_seq]
    t = b * s1
    bf = torch.bfloat16

    def uni(shape, dtype):
        return (torch.rand(shape, generator=g, dtype=torch.float32) * 2 - 1).to(dtype)

    x = uni([t, h], bf)
    q_norm = torch.randint(-128, 128, [t, q_lora_rank], generator=g, dtype=torch.int8)
    q_norm_scale = uni([t, 1], torch.float32)
    w_qb = torch.randint(-128, 128, [q_lora_rank, n_heads * head_dim], generator=g, dtype=torch.int8)
    w_qb_scale = uni([n_heads * head_dim, 1], torch.float32)
    wk = uni([h, head_dim], bf)
    w_proj = uni([h, n_heads], bf)
    if affine_ln:
        gamma, beta = uni([head_dim], bf), uni([head_dim], bf)
    else:
        gamma, beta = torch.ones([head_dim], dtype=bf), torch.zeros([head_dim], dtype=bf)
    ang = torch.rand([t, rope_dim], generator=g, dtype=torch.float32) * (2 * math.pi)
    cos, sin = torch.cos(ang).to(bf), torch.sin(ang).to(bf)
    hq, hk = uni([head_dim, head_dim], bf), uni([head_dim, head_dim], bf)
    block_num, table = gen_block_table(act, block_size, g, shuffle=True)
    k_cache = torch.randint(-128, 128, [block_num, block_size, 1, head_dim], generator=g, dtype=torch.int8)
    k_cache_scale = uni([block_num, block_size, 1, 1], torch.float16)
    idx = torch.empty([b, s1], dtype=torch.int64)
    for i in range(b):
        for j in range(s1):
            pos = act[i] - s1 + j
            idx[i, j] = int(table[i, pos // block_size]) * block_size + pos % block_size
    return IndexerPrologInputs(b=b, s1=s1, block_size=block_size, block_num=block_num, act_seq=act, x=x,
                               q_norm=q_norm, q_norm_scale=q_norm_scale, w_qb=w_qb, w_qb_scale=w_qb_scale,
                               wk=wk, w_proj=w_proj, ln_gamma_k=gamma, ln_beta_k=beta, cos_idx_rope=cos,
                               sin_idx_rope=sin, hadamard_q=hq, hadamard_k=hk, k_cache=k_cache,
                               k_cache_scale=k_cache_scale, k_cache_index=idx.reshape(t), block_table=table)


@dataclass
class MlaPrologInputs:
    b: int
    s1: int
    block_size: int
    block_num: int
    act_seq: List[int]
    token_x: torch.Tensor        # [T, h]                       bf16
    w_dq: torch.Tensor           # [h, q_lora_rank]             bf16
    w_uq_qr: torch.Tensor        # [q_lora_rank, N*192]         int8
    dequant_scale: torch.Tensor  # [N*192, 1]                   fp32
    w_uk: torch.Tensor           # [N, 128, 512]                bf16
    w_dkv_kr: torch.Tensor       # [h, 576]                     bf16
    gamma_cq: torch.Tensor       # [q_lora_rank]                bf16
    gamma_ckv: torch.Tensor      # [512]                        bf16
    cos: torch.Tensor            # [T, 64]                      bf16
    sin: torch.Tensor            # [T, 64]                      bf16
    cache_index: torch.Tensor    # [T]                          int64
    kv_cache: torch.Tensor       # [NB, bs, 1, 512]             int8   (updated in place)
    kr_cache: torch.Tensor       # [NB, bs, 1, 64]              bf16   (updated in place)
    k_scale_cache: torch.Tensor  # [NB, bs, 1, 4]               fp32   (updated in place)
    block_table: torch.Tensor    # [B, MB]                      int32

    def input_tensors(self):
        return (self.token_x, self.w_dq, self.w_uq_qr, self.dequant_scale, self.w_uk, self.w_dkv_kr, self.gamma_cq,
                self.gamma_ckv, self.cos, self.sin, self.cache_index, self.kv_cache, self.kr_cache, self.k_scale_cache)

    def to(self, device) -> "MlaPrologInputs":
        kw = dict(self.__dict__)
        for k, v in kw.items():
            if isinstance(v, torch.Tensor):
                kw[k] = v.to(device)
        return MlaPrologInputs(**kw)


def gen_mla_prolog_inputs(b: int, s1: int, act_seq: Sequence[int], seed: int = 0, h: int = 7168,
                          q_lora_rank: int = 1536, n_heads: int = 128, block_size: int = BLOCK_SIZE) -> MlaPrologInputs:
    """Value ranges of the reference generator: x, gammas uniform in (-1, 1), weights in (-0.1, 0.1) (w_uqqr
    quantised per output channel to int8), cos/sin in (-0.1, 0.1); caches filled with random rows."""
    g = torch.Generator().manual_seed(seed)
    act = [int(a) for a in act_seq]
    t = b * s1
    bf = torch.bfloat16
    d_nope, d_rope, kv_rank = 128, ROPE_DIM, KV_LORA_RANK

    def uni(shape, lim, dtype):
        return ((torch.rand(shape, generator=g, dtype=torch.float32) * 2 - 1) * lim).to(dtype)

    x = uni([t, h], 1.0, bf)
    w_dq = uni([h, q_lora_rank], 0.1, bf)
    wq = uni([q_lora_rank, n_heads * (d_nope + d_rope)], 0.1, torch.float32)
    amax = wq.abs().amax(dim=0, keepdim=True)
    sq = 127.0 / amax
    w_uq_qr = torch.round(wq * sq).to(torch.int8)
    dequant_scale = (1.0 / sq).reshape(-1, 1).contiguous()
    w_uk = uni([n_heads, d_nope, kv_rank], 0.1, bf)
    w_dkv_kr = uni([h, kv_rank + d_rope], 0.1, bf)
    gamma_cq, gamma_ckv = uni([q_lora_rank], 1.0, bf), uni([kv_rank], 1.0, bf)
    cos, sin = uni([t, d_rope], 0.1, bf), uni([t, d_rope], 0.1, bf)
    block_num, table = gen_block_table(act, block_size, g, shuffle=True)
    kv_cache = torch.randint(-127, 128, [block_num, block_size, 1, kv_rank], generator=g, dtype=torch.int8)
    kr_cache = uni([block_num, block_size, 1, d_rope], 1.0, bf)
    k_scale_cache = 0.005 + 0.015 * torch.rand([block_num, block_size, 1, 4], generator=g, dtype=torch.float32)
    idx = torch.empty([b, s1], dtype=torch.int64)
    for i in range(b):
        for j in range(s1):
            pos = act[i] - s1 + j
            idx[i, j] = int(table[i, pos // block_size]) * block_size + pos % block_size
    return MlaPrologInputs(b=b, s1=s1, block_size=block_size, block_num=block_num, act_seq=act, token_x=x, w_dq=w_dq,
                           w_uq_qr=w_uq_qr, dequant_scale=dequant_scale, w_uk=w_uk, w_dkv_kr=w_dkv_kr,
                           gamma_cq=gamma_cq, gamma_ckv=gamma_ckv, cos=cos, sin=sin, cache_index=idx.reshape(t),
                           kv_cache=kv_cache, kr_cache=kr_cache, k_scale_cache=k_scale_cache, block_table=table)


def config_lengths(cfg: int, seed: int = 0) -> List[int]:
    """Per-sequence KV lengths of the benchmark configurations 0-4."""
    g = torch.Generator().manual_seed(1000 + seed)
    if cfg == 0:
        return [4096]
    if cfg == 1:
        return [32768] * 4
    if cfg == 2:
        return torch.randint(8192, 65537, [32], generator=g).tolist()
    if cfg == 3:
        return torch.randint(4096, 32769, [64], generator=g).tolist()
    if cfg == 4:
        return [4096]
    raise ValueError(cfg)
