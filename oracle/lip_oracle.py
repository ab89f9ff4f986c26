"""CPU oracle for the quantized lightning-indexer prolog (projection stage).

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Restates the torch golden ``indexer_prolog`` of the reference example
(examples/models/deepseek_v32_exp/deepseekv32_lightning_indexer_prolog_quant.py:216-281
with its helpers ``layer_norm`` :170-177, ``quant_int8`` :180-192, ``rotate_half``
:195-198, ``single_rope`` :201-213, ``scatter_update_pa_bsnd`` :156-167; operator-side
statement examples/models/deepseek_v32_exp/lightning_indexer_prolog_quant_impl.py:325-504)
and fixes what the golden leaves to its libraries -- the order of every fp32 sum -- so that
a bit-exact comparison is meaningful.  All products below are products of two bf16 values
and therefore exact in fp32, so each sum is defined by its order alone (a fused
multiply-add and a multiply followed by an add give the same bits).

    query path, token t, head n, channel c (column ``n*128 + c`` of ``w_idx_qb``)
      acc   = sum_k int32(q_norm[t,k]) * int32(w_qb[k,col])                 exact  (:241)
      q     = bf16(rn32(rn32(float(acc) * q_norm_scale[t]) * w_qb_scale[col]))     (:242-245)
      q[0:64] = bf16(rn32(q*cos + rotate_half(q)*sin))     fp32, exact products    (:247)
      y[j]  = bf16(sum_{i=0..127} q[i] * H_q[i,j])         i ascending from 0.0    (:251)
      quant_int8(y) per (t, n)                                                     (:252)
    key path, token t
      k     = blocked_dot(x[t,:], w_idx_k)                                         (:255)
      k     = bf16(layer_norm(k))  with ``pair_tree_sum`` for both means           (:256)
      rope on the first 64 channels, y = bf16(sequential sum with H_k)             (:257-262)
      quant_int8(y); int8 row and fp16 scale written at row cache_index[t]         (:263-269)
    weights, token t
      w     = fp16(rn32(rn32(float(bf16(blocked_dot(x[t,:], w_idx_proj))) * f32(n**-0.5))
                        * f32(d**-0.5)))                                           (:272-275)

    blocked_dot   -- the reduction axis is cut into blocks of 64; a block is summed in
                     ascending order starting from 0.0; eight consecutive block sums are added
                     in ascending order (from 0.0) into a group sum; group sums are added in
                     ascending order (from 0.0).
    pair_tree_sum -- 128 values: adjacent pairs are added, then adjacent pairs of those
                     sums, ... (a balanced binary tree over neighbours).
    quant_int8    -- amax = max|y|; s = rn32(127/amax); out = int8(rint(rn32(y*s)));
                     dequant scale = fp16(rn32(1/s)).  The golden's detour through bf16
                     and trunc (:188) is the identity on integers up to 127.

One deliberate definition: a row with amax == 0 gives NaN in the golden (0 * inf); here
its int8 row is 0 and its scale is 0.

Pinning (tests/test_oracle_lip.py): integer matmul against Python integers; bf16 rounding
against an independent integer-arithmetic statement; rope against a float64 rotation of
(i, i+32) pairs and the identity at angle 0; the sequential Hadamard sum against exact
rational arithmetic on small cases, the identity matrix, and an order-sensitive vector;
layer norm against float64 statistics; quant_int8 known answers (the maximum maps to
+-127, scale*127 ~ amax); scatter touches exactly the rows named by cache_index; and the
whole function against :func:`indexer_prolog_library_order` -- the golden written with
torch.matmul/torch.mean, i.e. with the library's summation order -- at the reference's
own tolerances (deepseekv32_lightning_indexer_prolog_quant.py:424-428).
"""
from __future__ import annotations

import numpy as np
import torch

__all__ = [
    "BLOCK_K",
    "bf16_round",
    "blocked_dot",
    "pair_tree_sum",
    "q_linear",
    "rope_first",
    "hadamard_seq",
    "quant_int8",
    "layer_norm_fixed",
    "indexer_prolog_ref",
    "indexer_prolog_library_order",
]

BLOCK_K = 64
GROUP_BLOCKS = 8
F32 = np.float32


def _f32(t) -> np.ndarray:
    if isinstance(t, torch.Tensor):
        return t.detach().cpu().to(torch.float32).numpy()
    return np.asarray(t, dtype=F32)


def bf16_round(x: np.ndarray) -> np.ndarray:
    """fp32 -> nearest bf16 (ties to even), returned as fp32. Finite inputs."""
    x = np.ascontiguousarray(x, dtype=F32)
    u = x.view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(F32).reshape(x.shape)


def blocked_dot(x: np.ndarray, w: np.ndarray, block: int = BLOCK_K, group: int = GROUP_BLOCKS) -> np.ndarray:
    """[T,K] x [K,N] -> [T,N] fp32 in the fixed order stated in the module docstring."""
    x = np.asarray(x, F32)
    w = np.asarray(w, F32)
    t, k = x.shape
    assert k % block == 0 and w.shape[0] == k
    nb = k // block
    xb = x.reshape(t, nb, block)
    wb = w.reshape(nb, block, -1)
    part = np.zeros((t, nb, w.shape[1]), F32)
    for i in range(block):
        part = part + xb[:, :, i, None] * wb[None, :, i, :]
    total = np.zeros((t, w.shape[1]), F32)
    for g0 in range(0, nb, group):
        gsum = np.zeros((t, w.shape[1]), F32)
        for c in range(g0, min(g0 + group, nb)):
            gsum = gsum + part[:, c, :]
        total = total + gsum
    return total


def pair_tree_sum(v: np.ndarray) -> np.ndarray:
    """Balanced binary tree over neighbours along the last axis (length a power of two)."""
    v = np.asarray(v, F32)
    while v.shape[-1] > 1:
        v = v[..., 0::2] + v[..., 1::2]
    return v[..., 0]


def q_linear(q_norm: np.ndarray, w_qb: np.ndarray) -> np.ndarray:
    """Exact int8 x int8 matmul, [T,K] x [K,N] -> int32 (|sum| <= K * 2**14 < 2**31)."""
    # through the float64 matrix product: every product is below 2**14 and every partial sum below 2**31, all
    # exactly representable, so the sum is exact whatever order the library takes (an integer matmul in
    # numpy is the same numbers, two orders of magnitude slower)
    acc = q_norm.astype(np.float64) @ w_qb.astype(np.float64)
    return acc.astype(np.int64).astype(np.int32)


def rope_first(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """x [T, ..., 128] bf16-valued fp32; rotates channels 0..63 with cos/sin [T, 64]; bf16 result."""
    x = np.array(x, dtype=F32, copy=True)
    r = cos.shape[-1]
    shape = [x.shape[0]] + [1] * (x.ndim - 2) + [r]
    c = cos.reshape(shape)
    s = sin.reshape(shape)
    xr = x[..., :r]
    rot = np.concatenate([-xr[..., r // 2:], xr[..., :r // 2]], axis=-1)
    x[..., :r] = bf16_round(xr * c + rot * s)
    return x


def hadamard_seq(a: np.ndarray, h: np.ndarray) -> np.ndarray:
    """y[..., j] = sum_i a[..., i] * h[i, j], i ascending, fp32; bf16 result."""
    a = np.asarray(a, F32)
    h = np.asarray(h, F32)
    acc = np.zeros(a.shape[:-1] + (h.shape[1],), F32)
    for i in range(h.shape[0]):
        acc = acc + a[..., i, None] * h[i]
    return bf16_round(acc)


def quant_int8(y: np.ndarray):
    """Per-row symmetric int8 quantisation of bf16-valued fp32 rows -> (int8 rows, fp16 scales)."""
    y = np.asarray(y, F32)
    amax = np.max(np.abs(y), axis=-1, keepdims=True)
    ok = amax > 0
    safe = np.where(ok, amax, F32(1.0)).astype(F32)
    s = (F32(127.0) / safe).astype(F32)
    q = np.rint((y * s).astype(F32)).astype(np.int32)
    deq = (F32(1.0) / s).astype(F32)
    q = np.where(ok, q, 0).astype(np.int8)
    deq = np.where(ok, deq, F32(0.0)).astype(np.float16)
    return q, deq[..., 0]


def layer_norm_fixed(x: np.ndarray, gamma: np.ndarray, beta: np.ndarray, eps: float) -> np.ndarray:
    """fp32 layer norm over 128 channels with tree-ordered means; bf16 result."""
    x = np.asarray(x, F32)
    n = F32(x.shape[-1])
    mean = (pair_tree_sum(x) / n).astype(F32)[..., None]
    d = (x - mean).astype(F32)
    var = (pair_tree_sum((d * d).astype(F32)) / n).astype(F32)[..., None]
    std = np.sqrt((var + F32(eps)).astype(F32)).astype(F32)
    r = (d / std).astype(F32)
    return bf16_round(((r * gamma).astype(F32) + beta).astype(F32))


def indexer_prolog_ref(x, q_norm, q_norm_scale, w_qb, w_qb_scale, wk, w_proj, ln_gamma_k, ln_beta_k,
                       cos_idx_rope, sin_idx_rope, hadamard_q, hadamard_k, k_cache, k_cache_scale,
                       k_cache_index, eps: float = 1e-6):
    """Returns dict(q_int8 [T,N,128] int8, q_scale [T,N] fp16, k_cache, k_cache_scale (updated
    copies), weights [T,N] fp16, plus the int8 key rows and scales before the scatter)."""
    xf = _f32(x)
    t = xf.shape[0]
    d = hadamard_q.shape[0]
    n_heads = w_proj.shape[1]
    cos = _f32(cos_idx_rope)
    sin = _f32(sin_idx_rope)

    acc = q_linear(q_norm.cpu().numpy(), w_qb.cpu().numpy())                       # [T, N*d]
    qf = (acc.astype(F32) * _f32(q_norm_scale).reshape(t, 1)).astype(F32)
    qf = (qf * _f32(w_qb_scale).reshape(1, -1)).astype(F32)
    q = bf16_round(qf).reshape(t, n_heads, d)
    q = rope_first(q, cos, sin)
    q_int8, q_scale = quant_int8(hadamard_seq(q, _f32(hadamard_q)))

    k = blocked_dot(xf, _f32(wk))
    k = layer_norm_fixed(k, _f32(ln_gamma_k), _f32(ln_beta_k), eps)
    k = rope_first(k, cos, sin)
    k_int8, k_scale = quant_int8(hadamard_seq(k, _f32(hadamard_k)))

    kc = k_cache.cpu().numpy().copy()
    ks = k_cache_scale.cpu().numpy().copy()
    kc2 = kc.reshape(-1, d)
    ks2 = ks.reshape(-1)
    idx = k_cache_index.cpu().numpy().reshape(-1).astype(np.int64)
    for i in range(t):
        if 0 <= idx[i] < kc2.shape[0]:
            kc2[idx[i]] = k_int8[i]
            ks2[idx[i]] = k_scale[i]

    w = bf16_round(blocked_dot(xf, _f32(w_proj)))
    w = (w * F32(n_heads ** -0.5)).astype(F32)
    w = (w * F32(d ** -0.5)).astype(F32).astype(np.float16)

    return {"q_int8": q_int8, "q_scale": q_scale, "k_cache": kc, "k_cache_scale": ks, "weights": w,
            "k_int8": k_int8, "k_scale": k_scale}


def indexer_prolog_library_order(x, q_norm, q_norm_scale, w_qb, w_qb_scale, wk, w_proj, ln_gamma_k,
                                 ln_beta_k, cos_idx_rope, sin_idx_rope, hadamard_q, hadamard_k,
                                 eps: float = 1e-6):
    """The golden's statements with torch's own matmul / mean (summation order left to the library).
    Returns q_int8, q_scale, k_int8, k_scale, weights as torch tensors -- a second, independent
    evaluation used only to check the fixed-order oracle at the reference's tolerances."""
    t = x.shape[0]
    d = hadamard_q.shape[0]
    n = w_proj.shape[1]
    r = cos_idx_rope.shape[1]
    bf = torch.bfloat16

    def rope(v, cos, sin):
        vf = v.float()
        v1, v2 = vf.chunk(2, dim=-1)
        return (vf * cos + torch.cat((-v2, v1), dim=-1) * sin).to(bf)

    def quant(v):
        vf = v.float()
        amax = vf.abs().amax(dim=-1, keepdim=True)
        s = 127.0 / amax
        q = torch.round(vf * s).to(torch.int32).to(torch.int8)
        return q, (1.0 / s).to(torch.float16)

    cos = cos_idx_rope.float()
    sin = sin_idx_rope.float()
    q = torch.matmul(q_norm.to(torch.int32), w_qb.to(torch.int32)).float()
    q = (q * q_norm_scale.reshape(t, 1).float()) * w_qb_scale.reshape(1, -1).float()
    q = q.reshape(t, n, d).to(bf)
    q = torch.cat([rope(q[..., :r], cos[:, None, :], sin[:, None, :]), q[..., r:]], dim=-1)
    q = torch.matmul(q.float(), hadamard_q.float()).to(bf)
    q_int8, q_scale = quant(q)

    k = torch.matmul(x.float(), wk.float())
    mean = k.mean(dim=-1, keepdim=True)
    var = ((k - mean) ** 2).mean(dim=-1, keepdim=True)
    k = ((k - mean) / torch.sqrt(var + eps) * ln_gamma_k.float() + ln_beta_k.float()).to(bf)
    k = torch.cat([rope(k[..., :r], cos, sin), k[..., r:]], dim=-1)
    k = torch.matmul(k.float(), hadamard_k.float()).to(bf)
    k_int8, k_scale = quant(k)

    w = torch.matmul(x.float(), w_proj.float()).to(bf).float()
    w = (w * (n ** -0.5) * (d ** -0.5)).to(torch.float16)
    return q_int8, q_scale[..., 0], k_int8, k_scale[..., 0], w
