"""The HIP backend put through the reference's known-answer groups directly (not only through the
oracle): quantisation, half-precision arithmetic, the cast vectors, division by zero and the NaN
rules, integer extras and pow, the sums of ones, threefry, and the complex, bool, regression,
high-rank (rank 32) and fp8 groups of backend_contract.ml. Data: tests/golden/reference_vectors.json."""

import numpy as np
import pytest

import contract_groups as cg
from helpers import encode
from raven_amd import dtype as dt

pytestmark = pytest.mark.gpu

INT_DTYPES = [dt.int8, dt.uint8, dt.int16, dt.uint16, dt.int32, dt.uint32, dt.int64, dt.uint64]


def test_quantize_vectors(hip):
    cg.quantize(hip)


def test_half_binary_vectors(hip):
    cg.half_binary(hip)


def test_cast_vectors(hip):
    cg.cast_vectors(hip)


def test_zero_division_and_nan_rules(hip):
    cg.zero_division_and_nan_rules(hip)


def test_int_extra_and_pow(hip):
    cg.int_extra_and_pow(hip, INT_DTYPES)


def test_sums_of_ones(hip, oracle):
    cg.sums_of_ones(hip, lambda d: encode(np.array([1.0]), d, oracle))


def test_threefry_known_answers(hip):
    cg.threefry(hip)


def test_complex_group(hip):
    cg.complex_group(hip)


def test_bool_group(hip):
    cg.bool_group(hip)


def test_regression_group(hip):
    cg.regression_group(hip)


def test_highrank_group(hip):
    cg.highrank_group(hip)


def test_fp8_group(hip):
    cg.fp8_group(hip)
