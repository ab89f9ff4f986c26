"""CPU oracle for the quantized MLA prolog (bf16 down-projections, int8 query up-projection,
int8 latent KV with four fp32 scales per token -- the variant whose caches the sparse
attention of this path reads).

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Restates the torch golden ``mla_prolog_quant_v32_compute`` of the reference example
(examples/models/deepseek_v32_exp/deepseekv32_mla_prolog_quant.py:137-282 with its helpers
``rms_norm`` :35-51, ``scatter_update`` :54-69, ``rotate_half`` :72-76,
``apply_rotary_pos_emb_v2`` :79-104, ``quant`` :107-125) for ``is_quant_a = False``,
``is_quant_b = True``, no smoothing, cache mode PA_BSND -- the reference's enabled case
(:790-834); operator-side statement examples/models/deepseek_v32_exp/
mla_prolog_quant_impl.py:502-707.  As in the indexer-prolog oracle the order of every fp32
sum is fixed here (all products are bf16 x bf16, exact in fp32):

    q_a      = bf16(blocked_dot(x, w_dq))                                       (:178-180)
    q_norm   = bf16(rms(q_a, gamma_cq, eps_cq)); per-token int8 + fp32 scale    (:182-191)
    q_b      = bf16(rn32(rn32(float(int32 q_norm . w_uqqr) * scale[t]) * w_qb_scale[col]))   (:192-203)
    q_nope'  = bf16(sum_{i=0..127} q_b[t,n,i] * w_uk[n,i,:]),  i ascending      (:209-216)
    q_rope   = rope(q_b[t,n,128:192])                                           (:253-260)
    kv_a     = bf16(blocked_dot(x, w_dkvkr))                                    (:229-233)
    ckv      = bf16(rms(kv_a[:, :512], gamma_ckv, eps_ckv)); int8 in four groups of 128
               with one fp32 scale each                                         (:239-246)
    k_rope   = rope(kv_a[:, 512:576])
    rows cache_index[t] of kv_cache / kr_cache / kv_quant_scale_cache rewritten  (:262-279)

    blocked_dot -- as in oracle/lip_oracle.py (blocks of 64, groups of 8 block sums).
    rms         -- y = rn32(rn32(v*v) * f32(1/n)); slab sums: the 128 values of each slab
                   of 128 channels as a balanced tree over neighbours; slab sums added in
                   ascending order from 0.0; d = sqrt(rn32(sum + eps));
                   out = bf16(rn32(rn32(v / d) * gamma)).  The golden has no epsilon
                   (:35-51), the operator adds it under the root
                   (mla_prolog_quant_impl.py:127-163): eps is a parameter here, 0 gives
                   the golden's statement.
    rope        -- the 64 channels are first de-interleaved (even channels, then odd
                   channels: :93-97), then out = bf16(rn32(v*cos + rotate_half(v)*sin));
                   products exact, one rounding.
    quant       -- lip_oracle.quant_int8 with the scale kept in fp32.

Rows whose values are all zero quantise to zeros with scale 0 (the golden gives NaN).

Pinning (tests/test_oracle_mlap.py): the shared pieces are pinned in
tests/test_oracle_lip.py; here: rms against float64 and its sum order against exact
rationals; rope against a float64 rotation of the (2j, 2j+1) pairs and its channel
permutation by a known answer; per-group quantisation known answers; the absorb product
against exact rationals; scatter rows; and the whole function against
:func:`mla_prolog_library_order` (the golden with torch.matmul / torch.sum) at the
reference's tolerances (deepseekv32_mla_prolog_quant.py:668-692).
"""
from __future__ import annotations

import numpy as np
import torch

from .lip_oracle import F32, _f32, bf16_round, blocked_dot, pair_tree_sum, q_linear

__all__ = ["rms_fixed", "rope_deinterleaved", "quant_rows_f32", "absorb_seq", "mla_prolog_ref",
           "mla_prolog_library_order"]


def rms_fixed(v: np.ndarray, gamma: np.ndarray, eps: float) -> np.ndarray:
    """v [..., n] bf16-valued fp32 (n a multiple of 128) -> bf16-valued fp32."""
    v = np.asarray(v, F32)
    n = v.shape[-1]
    y = ((v * v).astype(F32) * F32(1.0 / n)).astype(F32)
    slabs = pair_tree_sum(y.reshape(v.shape[:-1] + (n // 128, 128)))          # [..., n/128]
    s = np.zeros(v.shape[:-1], F32)
    for j in range(n // 128):
        s = (s + slabs[..., j]).astype(F32)
    d = np.sqrt((s + F32(eps)).astype(F32)).astype(F32)[..., None]
    return bf16_round(((v / d).astype(F32) * np.asarray(gamma, F32)).astype(F32))


def rope_deinterleaved(v: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """v [T, ..., 64] bf16-valued; cos/sin [T, 64].  Even channels first, then odd; rotate-half."""
    v = np.asarray(v, F32)
    d = v.shape[-1]
    vp = np.concatenate([v[..., 0::2], v[..., 1::2]], axis=-1)
    shape = [v.shape[0]] + [1] * (v.ndim - 2) + [d]
    c = np.asarray(cos, F32).reshape(shape)
    s = np.asarray(sin, F32).reshape(shape)
    rot = np.concatenate([-vp[..., d // 2:], vp[..., :d // 2]], axis=-1)
    return bf16_round((vp * c + rot * s).astype(F32))


def quant_rows_f32(y: np.ndarray):
    """Per-row symmetric int8 quantisation; de-quantisation scale stays fp32."""
    y = np.asarray(y, F32)
    amax = np.max(np.abs(y), axis=-1, keepdims=True)
    ok = amax > 0
    safe = np.where(ok, amax, F32(1.0)).astype(F32)
    s = (F32(127.0) / safe).astype(F32)
    q = np.rint((y * s).astype(F32)).astype(np.int32)
    deq = (F32(1.0) / s).astype(F32)
    return np.where(ok, q, 0).astype(np.int8), np.where(ok, deq, F32(0.0)).astype(F32)[..., 0]


def absorb_seq(a: np.ndarray, w_uk: np.ndarray) -> np.ndarray:
    """a [T, N, 128], w_uk [N, 128, 512] -> bf16(sum_i a[t,n,i] * w_uk[n,i,:]), i ascending."""
    a = np.asarray(a, F32)
    w = np.asarray(w_uk, F32)
    acc = np.zeros(a.shape[:2] + (w.shape[2],), F32)
    for i in range(w.shape[1]):
        acc = acc + a[:, :, i, None] * w[None, :, i, :]
    return bf16_round(acc)


def mla_prolog_ref(token_x, w_dq, w_uq_qr, dequant_scale, w_uk, w_dkv_kr, gamma_cq, gamma_ckv, cos, sin, cache_index,
                   kv_cache, kr_cache, k_scale_cache, epsilon_cq: float = 0.0, epsilon_ckv: float = 0.0):
    """Returns dict(q_norm int8 [T,1536], q_norm_scale fp32 [T], query_nope bf16-valued fp32 [T,N,512],
    query_rope [T,N,64], kv_cache int8, kr_cache (fp32 values of bf16), k_scale_cache fp32 -- updated copies --
    and the per-token rows before the scatter)."""
    xf = _f32(token_x)
    t = xf.shape[0]
    n, d_nope, kv_rank = w_uk.shape
    d_rope = cos.shape[-1]
    cosf, sinf = _f32(cos).reshape(t, d_rope), _f32(sin).reshape(t, d_rope)

    q_a = bf16_round(blocked_dot(xf, _f32(w_dq)))
    q_norm, q_scale = quant_rows_f32(rms_fixed(q_a, _f32(gamma_cq), epsilon_cq))
    acc = q_linear(q_norm, w_uq_qr.cpu().numpy())
    q_b = (acc.astype(F32) * q_scale[:, None]).astype(F32)
    q_b = bf16_round((q_b * _f32(dequant_scale).reshape(1, -1)).astype(F32)).reshape(t, n, d_nope + d_rope)
    query_nope = absorb_seq(q_b[..., :d_nope], _f32(w_uk))
    query_rope = rope_deinterleaved(q_b[..., d_nope:], cosf, sinf)

    kv_a = bf16_round(blocked_dot(xf, _f32(w_dkv_kr)))
    ckv = rms_fixed(kv_a[:, :kv_rank], _f32(gamma_ckv), epsilon_ckv)
    k_int8, k_scales = quant_rows_f32(ckv.reshape(t, 4, kv_rank // 4))
    k_int8 = k_int8.reshape(t, kv_rank)
    k_rope = rope_deinterleaved(kv_a[:, kv_rank:], cosf, sinf)

    kvc = kv_cache.cpu().numpy().copy()
    krc = _f32(kr_cache).copy()
    ksc = k_scale_cache.cpu().numpy().astype(F32).copy()
    kv2, kr2, ks2 = kvc.reshape(-1, kv_rank), krc.reshape(-1, d_rope), ksc.reshape(-1, 4)
    idx = cache_index.cpu().numpy().reshape(-1).astype(np.int64)
    for i in range(t):
        if 0 <= idx[i] < kv2.shape[0]:
            kv2[idx[i]] = k_int8[i]
            kr2[idx[i]] = k_rope[i]
            ks2[idx[i]] = k_scales[i]
    return {"q_norm": q_norm, "q_norm_scale": q_scale, "query_nope": query_nope, "query_rope": query_rope,
            "kv_cache": kvc, "kr_cache": krc, "k_scale_cache": ksc, "k_int8": k_int8, "k_rope": k_rope,
            "k_scales": k_scales}


def mla_prolog_library_order(token_x, w_dq, w_uq_qr, dequant_scale, w_uk, w_dkv_kr, gamma_cq, gamma_ckv, cos, sin):
    """The golden's statements with torch's own matmul / sum (no epsilon, as the golden).  Returns q_norm,
    q_norm_scale, query_nope, query_rope, k_int8, k_rope, k_scales for the tokens (no scatter)."""
    bf = torch.bfloat16
    t = token_x.shape[0]
    n, d_nope, kv_rank = w_uk.shape
    d_rope = cos.shape[-1]

    def rms(v, gamma):
        vf = v.float()
        s = torch.sum(vf * vf * (1.0 / v.shape[-1]), dim=-1, keepdim=True)
        return ((vf / torch.sqrt(s)) * gamma.float()).to(bf)

    def quant(v):
        vf = v.float()
        amax = vf.abs().amax(dim=-1, keepdim=True)
        s = 127 / amax
        return torch.round(vf * s).to(torch.int32).to(torch.int8), 1 / s

    def rope(v, c, s):
        vf = v.float()
        sh = vf.shape
        vp = vf.reshape(sh[:-1] + (sh[-1] // 2, 2)).transpose(-1, -2).reshape(sh)
        rot = torch.cat((-vp[..., sh[-1] // 2:], vp[..., :sh[-1] // 2]), dim=-1)
        return (vp * c + rot * s).to(bf)

    cf, sf = cos.reshape(t, d_rope).float(), sin.reshape(t, d_rope).float()
    q_a = torch.matmul(token_x.float(), w_dq.float()).to(bf)
    q_norm, q_scale = quant(rms(q_a, gamma_cq))
    q_b = torch.matmul(q_norm.to(torch.int32), w_uq_qr.to(torch.int32)).float() * q_scale
    q_b = (q_b * dequant_scale.reshape(1, -1).float()).to(bf).reshape(t, n, d_nope + d_rope)
    qn = torch.matmul(q_b[..., :d_nope].permute(1, 0, 2).float(), w_uk.float()).to(bf).permute(1, 0, 2)
    qr = rope(q_b[..., d_nope:], cf[:, None, :], sf[:, None, :])
    kv_a = torch.matmul(token_x.float(), w_dkv_kr.float()).to(bf)
    ckv = rms(kv_a[:, :kv_rank], gamma_ckv)
    k_int8, k_scales = quant(ckv.reshape(t, 4, kv_rank // 4))
    kr = rope(kv_a[:, kv_rank:], cf, sf)
    return q_norm, q_scale[:, 0], qn, qr, k_int8.reshape(t, kv_rank), kr, k_scales.reshape(t, 4)
