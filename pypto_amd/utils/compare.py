"""Result comparators with the reference drivers' semantics.

* :func:`compare` -- examples/models/deepseek_v32_exp/utils/compare.py:23-130 of
  the reference: NaN/Inf in the tested tensor is an error; an element is an
  outlier when ``|t - ref| > atol + rtol * |ref|``; the tensors match when the
  number of outliers does not exceed ``round(max_error_ratio * numel)``.
* :func:`topk_idx_compare` -- examples/models/deepseek_v32_exp/
  deepseekv32_lightning_indexer_quant.py:272-314: rows of ``group`` entries are
  compared as sets over the positions that differ; a row passes when at most
  ``int(group * atol)`` expected indices are missing.
* :func:`attention_error_stats` -- the two figures the benchmark tolerance is
  stated in: max-abs error and mean-rel error (mean |t-ref| / mean |ref|).
"""
from __future__ import annotations

import torch


def compare(t: torch.Tensor, t_ref: torch.Tensor, name: str, atol: float, rtol: float,
            max_error_ratio: float = 0.005, max_error_count: int = 10) -> None:
    nan_count = int(torch.isnan(t).sum())
    inf_count = int(torch.isinf(t).sum())
    assert nan_count == 0 and inf_count == 0, f"{name}: {nan_count} NaN and {inf_count} Inf values"
    assert t.shape == t_ref.shape, f"{name}: shape {tuple(t.shape)} vs {tuple(t_ref.shape)}"
    assert t.dtype == t_ref.dtype, f"{name}: dtype {t.dtype} vs {t_ref.dtype}"
    assert t.device == t_ref.device, f"{name}: device {t.device} vs {t_ref.device}"
    threshold = round(max_error_ratio * t_ref.numel())
    tf, rf = t.to(torch.float32), t_ref.to(torch.float32)
    diff = (tf - rf).abs()
    bad = diff > (atol + rtol * rf.abs())
    n_bad = int(bad.sum())
    if n_bad > 0:
        pos = torch.nonzero(bad)[:max_error_count]
        lines = [f"{name}: {n_bad} outliers (allowed {threshold}); first {len(pos)}:"]
        for p in pos:
            idx = tuple(int(v) for v in p)
            lines.append(f"  {idx}: {float(tf[idx]):.8f} vs {float(rf[idx]):.8f}")
        print("\n".join(lines))
    max_diff = float(diff.max()) if diff.numel() else 0.0
    assert n_bad <= threshold, f"compare fail: {name}, max diff {max_diff:.8f}, outliers {n_bad} > {threshold}"


def topk_idx_compare(t: torch.Tensor, t_ref: torch.Tensor, name: str, atol: float, group: int) -> None:
    a = t.reshape(-1, group)
    r = t_ref.reshape(-1, group)
    assert a.shape == r.shape, f"{name}: shape {tuple(t.shape)} vs {tuple(t_ref.shape)}"
    allowed = int(group * atol)
    for row in range(a.shape[0]):
        mism = a[row] != r[row]
        if not bool(mism.any()):
            continue
        exp = set(a[row][mism].tolist())
        act = set(r[row][mism].tolist())
        missing = len(exp - act)
        assert missing <= allowed, f"compare fail: {name}, row {row}: {missing} indices differ (allowed {allowed})"


def attention_error_stats(t: torch.Tensor, t_ref: torch.Tensor):
    """(max_abs, mean_rel) with mean_rel = mean|t-ref| / mean|ref|."""
    tf, rf = t.to(torch.float32), t_ref.to(torch.float32)
    d = (tf - rf).abs()
    denom = float(rf.abs().mean())
    return float(d.max()), float(d.mean()) / (denom if denom > 0 else 1.0)
