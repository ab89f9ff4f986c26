from .compare import compare, topk_idx_compare, attention_error_stats  # noqa: F401
