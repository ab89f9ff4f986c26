"""The comparators restated from the reference drivers (examples/models/deepseek_v32_exp/utils/compare.py:23-130,
deepseekv32_lightning_indexer_quant.py:272-314), checked on cases small enough to count by hand.  What a
plausible mistake would change: ``>`` against ``>=`` at the bound, the bound taken from the tested tensor
instead of the reference, truncation instead of Python's ``round`` for the allowed count, Inf accepted where
the reference holds Inf too."""
import pytest
import torch

from pypto_amd.utils.compare import attention_error_stats, compare, topk_idx_compare


def test_outlier_bound_is_per_element_and_strict():
    ref = torch.tensor([1.0, 2.0, 4.0, 0.0])
    # bound per element: 0.5 + 0.25 * |ref| = 0.75, 1.0, 1.5, 0.5 (all exact in fp32)
    on_bound = ref + torch.tensor([0.75, -1.0, 1.5, -0.5])
    compare(on_bound, ref, "on the bound", 0.5, 0.25, max_error_ratio=0.0)           # equality is no outlier
    past = on_bound.clone()
    past[3] = -0.50001
    with pytest.raises(AssertionError, match="compare fail"):
        compare(past, ref, "just past", 0.5, 0.25, max_error_ratio=0.0)
    # the bound follows |ref|, not |t|: t = 3 against ref = 1 is off by 2 > 0.5 + 0.25 * 1 although 2 <= 0.5 + 0.25 * 6
    with pytest.raises(AssertionError, match="compare fail"):
        compare(torch.tensor([3.0]), torch.tensor([1.0]), "bound from the reference", 0.5, 0.25, max_error_ratio=0.0)
    # a small reference element gets a small bound: one global bound (atol + rtol * max|ref|) would pass this
    small = torch.tensor([100.0, 0.0])
    with pytest.raises(AssertionError, match="compare fail"):
        compare(small + torch.tensor([0.0, 5.0]), small, "small element", 0.1, 0.1, max_error_ratio=0.0)


def test_allowed_count_is_python_round_of_ratio_times_numel():
    ref = torch.zeros(300)
    t = ref.clone()
    t[:2] = 1.0                                  # two outliers
    compare(t, ref, "2 of 300 at 0.5 %", 1e-3, 0.0, max_error_ratio=0.005)       # round(1.5) == 2
    t[2] = 1.0                                   # three
    with pytest.raises(AssertionError, match="outliers 3 > 2"):
        compare(t, ref, "3 of 300 at 0.5 %", 1e-3, 0.0, max_error_ratio=0.005)
    # round half to even: round(0.5) == 0 and round(2.5) == 2, where rounding half up would allow 1 and 3
    ref100 = torch.zeros(100)
    one = ref100.clone()
    one[0] = 1.0
    with pytest.raises(AssertionError, match="outliers 1 > 0"):
        compare(one, ref100, "1 of 100 at 0.5 %", 1e-3, 0.0, max_error_ratio=0.005)
    ref500 = torch.zeros(500)
    three = ref500.clone()
    three[:3] = 1.0
    with pytest.raises(AssertionError, match="outliers 3 > 2"):
        compare(three, ref500, "3 of 500 at 0.5 %", 1e-3, 0.0, max_error_ratio=0.005)
    three[2] = 0.0
    compare(three, ref500, "2 of 500 at 0.5 %", 1e-3, 0.0, max_error_ratio=0.005)
    # ratio 0 allows nothing; the default ratio is 0.005
    compare(ref100, ref100, "identical", 0.0, 0.0, max_error_ratio=0.0)
    t200 = torch.zeros(200)
    t200[0] = 1.0
    compare(t200, torch.zeros(200), "default ratio", 1e-3, 0.0)                      # round(1.0) == 1


def test_nan_and_inf_in_the_tested_tensor_are_errors():
    ref = torch.tensor([1.0, float("inf"), 3.0])
    with pytest.raises(AssertionError, match="NaN"):
        compare(torch.tensor([1.0, 2.0, float("nan")]), torch.tensor([1.0, 2.0, 3.0]), "nan", 1.0, 1.0, 1.0)
    with pytest.raises(AssertionError, match="Inf"):
        compare(ref.clone(), ref, "inf equal to the reference's inf", 1.0, 1.0, 1.0)
    with pytest.raises(AssertionError, match="Inf"):
        compare(torch.tensor([1.0, -float("inf"), 3.0]), torch.tensor([1.0, 2.0, 3.0]), "-inf", 1.0, 1.0, 1.0)


def test_shape_and_dtype_must_agree():
    with pytest.raises(AssertionError, match="shape"):
        compare(torch.zeros(2, 3), torch.zeros(3, 2), "shape", 1.0, 1.0)
    with pytest.raises(AssertionError, match="dtype"):
        compare(torch.zeros(4), torch.zeros(4, dtype=torch.bfloat16), "dtype", 1.0, 1.0)


def test_integer_tensors_compare_by_value():
    # the int8 rule of the prolog drivers: atol 1, rtol 0 -- off by one passes, off by two is an outlier,
    # and 127 against -128 is 255 apart (no int8 wrap-around)
    ref = torch.tensor([10, -128, 127, 0], dtype=torch.int8)
    compare(torch.tensor([11, -127, 126, -1], dtype=torch.int8), ref, "off by one", 1.0, 0.0, max_error_ratio=0.0)
    with pytest.raises(AssertionError, match="compare fail"):
        compare(torch.tensor([12, -128, 127, 0], dtype=torch.int8), ref, "off by two", 1.0, 0.0, max_error_ratio=0.0)
    with pytest.raises(AssertionError, match="max diff 255"):
        compare(torch.tensor([10, 127, 127, 0], dtype=torch.int8), ref, "wrap", 1.0, 0.0, max_error_ratio=0.0)


def test_topk_idx_compare_counts_missing_indices_per_row():
    ref = torch.arange(40, dtype=torch.int32).reshape(2, 20)
    same_set = ref.clone()
    same_set[0] = ref[0].flip(0)                                   # another order, the same set: passes at atol 0
    topk_idx_compare(same_set, ref, "permuted", 0.0, 20)
    one_off = ref.clone()
    one_off[1, 3] = 999                                            # one index of row 1 replaced
    topk_idx_compare(one_off, ref, "one of 20 at 5 %", 0.05, 20)   # int(20 * 0.05) == 1 allowed
    with pytest.raises(AssertionError, match="row 1"):
        topk_idx_compare(one_off, ref, "one of 20 at 4.9 %", 0.049, 20)          # int(0.98) == 0
    two_off = one_off.clone()
    two_off[1, 7] = 998
    with pytest.raises(AssertionError, match="2 indices differ"):
        topk_idx_compare(two_off, ref, "two of 20 at 5 %", 0.05, 20)


def test_attention_error_stats_closed_form():
    ref = torch.tensor([1.0, -3.0, 0.0, 4.0])
    t = torch.tensor([1.5, -3.0, 0.25, 3.0])
    max_abs, mean_rel = attention_error_stats(t, ref)
    assert max_abs == 1.0
    assert mean_rel == pytest.approx((0.5 + 0.0 + 0.25 + 1.0) / (1.0 + 3.0 + 0.0 + 4.0))
