"""Pins R2 (compile-side requant parameter derivation) of the oracle and of the workload generators."""
import numpy as np

from oracle import oracle as orc
from torq_compiler_amd import workloads


def test_min_shift_normalisation_bounds():
    rng = np.random.default_rng(0)
    mult = rng.integers(1 << 30, (1 << 31) - 1, size=64).astype(np.int32)
    shift = rng.integers(36, 43, size=64).astype(np.int8)
    sb, sf = orc.derive_scale_bias(mult, shift, None, None, 0)
    assert sf == int(shift.min())
    scale = sb[1::2].astype(np.int64)
    d = (shift.astype(np.int64) - sf)
    # scale is the multiplier with its low (shift - min) bits dropped
    assert np.all(scale << d <= mult) and np.all(mult < (scale + 1) << d)
    assert np.all(sb[0::2] == 0)


def test_bias_folds_input_zero_point():
    w = np.array([[1, 2, 3], [-4, 5, -6]], dtype=np.int8)
    sb, sf = orc.derive_scale_bias(np.array([1 << 30, 1 << 30], dtype=np.int32), np.array([30, 31], dtype=np.int8),
                                   np.array([100, -100], dtype=np.int32), orc.per_channel_sum(w), -3)
    assert sf == 30
    assert sb.tolist() == [100 + 3 * 6, 1 << 30, -100 + 3 * -5, 1 << 29]


def test_negative_multiplier_uses_arithmetic_shift():
    sb, sf = orc.derive_scale_bias(np.array([-7, 1 << 30], dtype=np.int32), np.array([12, 10], dtype=np.int8), None, None, 0)
    assert sf == 10 and sb[1] == (-7 >> 2) and sb[3] == 1 << 30


def test_workload_generator_matches_oracle_derivation():
    rng = np.random.default_rng(4)
    w = rng.integers(-127, 128, size=(16, 8, 3, 3)).astype(np.int8)
    mult, shift = workloads.random_requant(rng, 16, True)
    tb = rng.integers(-(1 << 15), 1 << 15, size=16)
    sb_a, sf_a = workloads.derive_scale_bias(mult, shift, tb, w, -3)
    sb_b, sf_b = orc.derive_scale_bias(mult, shift, tb.astype(np.int32), orc.per_channel_sum(w), -3)
    assert sf_a == sf_b and np.array_equal(sb_a, sb_b)
    wa, sba, sfa = workloads.add_params(0.71838506, 0.65, -3, 7)
    wb, sbb, sfb = orc.derive_add_params(0.71838506, 0.65, -3, 7)
    assert np.array_equal(wa, wb) and np.array_equal(sba, sbb) and sfa == sfb
