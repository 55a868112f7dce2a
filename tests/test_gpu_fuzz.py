"""Differential tests on random cases (tests/fuzz_cases.py): a fixed number of seeded cases per entry-point family, small
enough to run in seconds.  The same generators run for minutes from the command line."""
import random

import pytest

import fuzz_cases

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [101, 102])
def test_random_slices_pack_and_unpack_like_numpy_indexing(seed):
    gen = random.Random(seed)
    for i in range(800):
        fuzz_cases.pack_case(gen, f"seed {seed} case {i}", max_bytes=2 << 20, max_span_bytes=32 << 20)


@pytest.mark.parametrize("seed", [201, 202])
def test_random_reduces_match_the_oracle(seed):
    gen = random.Random(seed)
    for i in range(300):
        fuzz_cases.reduce_case(gen, f"seed {seed} case {i}", max_numel=1 << 18)


@pytest.mark.parametrize("seed", [301, 302])
def test_random_fp8_buckets_match_the_oracle(seed):
    gen = random.Random(seed)
    for i in range(80):
        fuzz_cases.fp8_case(gen, f"seed {seed} case {i}", max_tensor=60000)


@pytest.mark.parametrize("seed", [401, 402])
def test_random_groups_of_views_pack_and_unpack_in_one_call(seed):
    gen = random.Random(seed)
    for i in range(200):
        fuzz_cases.many_case(gen, f"seed {seed} case {i}")


@pytest.mark.parametrize("seed", [501, 502])
def test_random_reduce_scatters_match_the_oracle(seed):
    gen = random.Random(seed)
    for i in range(200):
        fuzz_cases.scatter_case(gen, f"seed {seed} case {i}", max_len=1 << 16)
