"""first_occurrences on the device: integer work, bit-exact.

Checked against the definition (lower / upper bound of every value in the
sorted vector, -1/-1 when the value is absent), which the oracle states with
std::lower_bound / std::upper_bound and numpy states with searchsorted, and
against the example documented in the reference
(mops/src/internal/cuda_first_occurences.cuh:7-9 of lab-cosmo/mops).
"""
import numpy as np
import pytest

from tests import support

pytestmark = pytest.mark.gpu


def by_definition(index, n_out):
    values = np.arange(n_out)
    first = np.searchsorted(index, values, side="left").astype(np.int32)
    last = np.searchsorted(index, values, side="right").astype(np.int32)
    absent = first == last
    first[absent] = -1
    last[absent] = -1
    return np.stack([first, last])


def run(index, n_out, device):
    import torch

    import mops_amd

    tensor = torch.from_numpy(np.asarray(index, dtype=np.int32)).to(device)
    return mops_amd.first_occurrences(tensor, n_out).cpu().numpy()


def test_documented_example(device):
    out = run([0, 0, 0, 1, 1, 1, 2, 2], 3, device)
    assert out[0].tolist() == [0, 3, 6]
    assert out[1].tolist() == [3, 6, 8]


@pytest.mark.parametrize(
    "n_in,n_out,allow_empty",
    [(1, 1, False), (7, 3, True), (513, 40, True), (60000, 2000, False), (60000, 2000, True),
     (1000, 5000, True), (100000, 3, False), (4097, 4097, False)],
)  # fmt: skip
def test_matches_definition(oracle, device, n_in, n_out, allow_empty):
    rng = np.random.default_rng(n_in * 31 + n_out)
    index = support.segments(rng, n_out, n_in, allow_empty)
    expected = by_definition(index, n_out)
    # the oracle states the same definition in C++
    from_oracle = np.empty(2 * n_out, dtype=np.int32)
    oracle.cdll.mops_oracle_first_occurrences(index.ctypes.data, n_in, n_out, from_oracle.ctypes.data)
    assert np.array_equal(from_oracle.reshape(2, n_out), expected)
    assert np.array_equal(run(index, n_out, device), expected)


def test_gaps_at_both_ends_and_in_the_middle(device):
    index = np.array([3, 3, 4, 9, 9, 9], dtype=np.int32)
    assert np.array_equal(run(index, 12, device), by_definition(index, 12))


def test_empty_input(device):
    out = run(np.zeros(0, dtype=np.int32), 17, device)
    assert np.all(out == -1)


def test_every_element_is_written(device):
    """The result buffer needs no initialisation: poison it first."""
    import ctypes

    import torch

    from mops_amd._c_lib import device_library

    rng = np.random.default_rng(5)
    index = support.segments(rng, 300, 1000, True)
    tensor = torch.from_numpy(index).to(device)
    result = torch.full((2, 300), 12345, dtype=torch.int32, device=device)
    library = device_library()
    library.cdll.mops_amd_set_stream(ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream))
    library.cdll.mops_amd_set_synchronous(1)
    status = library.cdll.mops_amd_first_occurrences(tensor.data_ptr(), 1000, 300, result.data_ptr())
    assert status == 0
    assert np.array_equal(result.cpu().numpy(), by_definition(index, 300))
