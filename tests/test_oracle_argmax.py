"""Oracle pin for the greedy token choice: the reference's own unit-test vectors of
argmax_token (src/engine/executor_step.rs:2191-2325)."""
import numpy as np

NAN = float("nan")


def test_reference_vectors(oracle):
    am = oracle.argmax_token
    assert am([0.1, 0.2, 0.5, 0.9, 0.3]) == 3            # argmax_token_basic
    assert am([42.0]) == 0                               # argmax_token_single
    assert am([]) is None                                # argmax_token_empty_returns_none
    assert am([1.0, 5.0, 5.0, 2.0]) == 2                 # argmax_token_tie_returns_last
    assert am([3.0, 3.0, 3.0]) == 2                      # argmax_token_all_equal
    assert am([0.1, 0.2, 0.3, 0.4, 99.0]) == 4           # argmax_token_last_is_max
    assert am([-10.0, -5.0, -20.0]) == 1                 # argmax_token_with_negative
    assert am([NAN, 1.0]) == 1                           # argmax_token_with_nan
    assert am([NAN, NAN, NAN]) is None                   # argmax_token_all_nan_returns_none
    big = np.zeros(10000, np.float32)
    big[7777] = 1.0
    assert am(big) == 7777                               # argmax_token_large_slice


def test_what_partial_cmp_implies(oracle):
    am = oracle.argmax_token
    assert am([0.0, -0.0]) == 1 and am([-0.0, 0.0]) == 1  # the two zeros compare equal: the last wins
    assert am([float("-inf"), NAN]) == 0                   # -inf is a value, NaN is not
    assert am([float("inf"), 1.0, float("inf")]) == 2
    assert am([NAN, -1.0, NAN, -1.0, NAN]) == 3
