"""The reference-held vectors of tests/golden/reference_vectors.json run through the HIP path."""

import pytest
import torch

from tests import golden_checks as G
from tests.adapters import HipImpl

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def impl(device):
    return HipImpl(device)


@pytest.mark.parametrize("name", [n for n in G.vector_set_names() if not n.startswith("bfloat16")])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32], ids=["f16", "f32"])
def test_vector_sets(impl, name, dtype):
    G.check_vector_set(impl, name, dtype)


@pytest.mark.parametrize("name", [n for n in G.vector_set_names() if n.startswith("bfloat16")])
def test_vector_sets_bfloat16(impl, name):
    G.check_vector_set(impl, name, torch.bfloat16)


def test_block_quant_table(impl):
    G.check_block_quant(impl)


def test_docstring_examples(impl):
    G.check_docstring_examples(impl)


def test_clipped_scale_gradient(impl):
    G.check_clipped_scale_gradient(impl)


def test_minmax_encodings(impl):
    G.check_minmax_encodings(impl)


def test_histogram_merges(impl):
    G.check_histogram_merges(impl)


def test_sqnr_uniform(impl):
    G.check_sqnr_uniform(impl)


def test_sqnr_outlier(impl):
    G.check_sqnr_outlier(impl)


def test_sqnr_brute_force(impl):
    G.check_sqnr_brute_force(impl)


def test_percentile(impl):
    G.check_percentile(impl)
