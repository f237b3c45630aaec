"""The oracle against the reference's complex, bool, regression, high-rank and fp8 contract groups
(backend_contract.ml:2319-2700, 3012-3122), transcribed as data into
tests/golden/reference_vectors.json. The same functions run against the HIP backend in
tests/test_gpu_contract_groups.py."""

import contract_groups as cg


def test_complex_group(oracle):
    cg.complex_group(oracle)


def test_bool_group(oracle):
    cg.bool_group(oracle)


def test_regression_group(oracle):
    cg.regression_group(oracle)


def test_highrank_group(oracle):
    cg.highrank_group(oracle)


def test_fp8_group(oracle):
    cg.fp8_group(oracle)


def test_the_shared_forms_of_the_older_groups(oracle):
    """quantize / half arithmetic / cast / zero division / int extras / threefry in the form the GPU
    test calls them (tests/test_oracle_pins.py holds the oracle's own, older copies)."""
    from raven_amd import dtype as dt

    cg.quantize(oracle)
    cg.half_binary(oracle)
    cg.cast_vectors(oracle)
    cg.zero_division_and_nan_rules(oracle)
    cg.int_extra_and_pow(oracle, [dt.int8, dt.uint8, dt.int16, dt.uint16, dt.int32, dt.uint32, dt.int64, dt.uint64])
    cg.threefry(oracle)
