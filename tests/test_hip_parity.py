"""Parity of the HIP kernels with the CPU oracle, through the device C ABI.

Bar (from the north star): max|x - ref| / max|ref| <= 1e-12 in float64 and
<= 1e-5 in float32, for outputs and every gradient. Small seeded cases cover
the shapes and edge cases of the reference's own tests (empty segments,
ragged sizes, every subset of requested gradients, unsorted SAP output
index); the BASELINE configurations are checked at full size against the
oracle and through size-independent properties (linearity, adjoint identity,
run-to-run bit reproducibility).
"""
import itertools

import numpy as np
import pytest

from tests import support
from tests.support import OPS, assert_close, cpu_forward, cpu_vjp, hip_forward, hip_vjp, to_device

pytestmark = pytest.mark.gpu

DTYPES = [np.float32, np.float64]

# name -> builder(seed, dtype); shapes chosen to hit partial tiles, sizes
# that are not multiples of the wavefront, and segments of very unequal length
CASES = {
    "hpe": {
        "tiny": lambda s, d: support.hpe_case(s, d, I=5, nA=3, J=7, K=2),
        "ragged": lambda s, d: support.hpe_case(s, d, I=203, nA=17, J=301, K=3),
        "order0": lambda s, d: support.hpe_case(s, d, I=70, nA=4, J=33, K=0),
        "order1": lambda s, d: support.hpe_case(s, d, I=70, nA=4, J=33, K=1),
        "order6": lambda s, d: support.hpe_case(s, d, I=130, nA=9, J=90, K=6),
        # (orders 7 to 10, the highest the reference takes, mops/src/hpe/cpu.tpp:77-130: the kernels with the order as a
        # run-time value)
        "order7": lambda s, d: support.hpe_case(s, d, I=90, nA=8, J=60, K=7),
        "order10": lambda s, d: support.hpe_case(s, d, I=77, nA=6, J=45, K=10),
        # (more features than a workgroup's LDS holds a row of: the kernels that read A from global memory)
        "many_features": lambda s, d: support.hpe_case(s, d, I=40, nA=16000, J=300, K=3),
        "many_rows": lambda s, d: support.hpe_case(s, d, I=70000, nA=12, J=40, K=3),
        "wide": lambda s, d: support.hpe_case(s, d, I=64, nA=2000, J=500, K=4),
    },
    "sap": {
        "tiny": lambda s, d: support.sap_case(s, d, I=3, nA=2, nB=2, K=5, nO=3),
        "ragged": lambda s, d: support.sap_case(s, d, I=333, nA=13, nB=7, K=211, nO=20),
        "unsorted": lambda s, d: support.sap_case(s, d, I=130, nA=6, nB=9, K=150, nO=11, sort_output=False),
        "wide": lambda s, d: support.sap_case(s, d, I=100, nA=70, nB=50, K=400, nO=300),
        "one_product": lambda s, d: support.sap_case(s, d, I=65, nA=3, nB=3, K=1, nO=4),
        # (more than 2048 entries on the matrix-core path: eight entries per thread while the dense table is built;
        # many entries per cell, added in ascending entry order)
        "table_of_2500": lambda s, d: support.sap_case(s, d, I=500, nA=9, nB=9, K=2500, nO=9),
        "table_of_8192_unsorted": lambda s, d: support.sap_case(s, d, I=300, nA=4, nB=5, K=8192, nO=6, sort_output=False),
        "table_of_2049": lambda s, d: support.sap_case(s, d, I=300, nA=13, nB=7, K=2049, nO=20),
    },
    "opsa": {
        "tiny": lambda s, d: support.opsa_case(s, d, J=6, K=2, L=3, n_out=4, allow_empty=True),
        "ragged": lambda s, d: support.opsa_case(s, d, J=1000, K=13, L=20, n_out=37, allow_empty=True),
        "long_segments": lambda s, d: support.opsa_case(s, d, J=3000, K=5, L=7, n_out=6),
        "wide": lambda s, d: support.opsa_case(s, d, J=400, K=40, L=33, n_out=21, allow_empty=True),
        # (more than 64 columns of A: the vjp whose rows of grad_output are staged in LDS)
        "tall": lambda s, d: support.opsa_case(s, d, J=400, K=70, L=33, n_out=21, allow_empty=True),
        "sixty_four_by_sixty_four": lambda s, d: support.opsa_case(s, d, J=500, K=64, L=64, n_out=25, allow_empty=True),
        "mostly_empty": lambda s, d: support.opsa_case(s, d, J=20, K=4, L=4, n_out=300, allow_empty=True),
        "pooling": lambda s, d: support.opsa_case(s, d, J=5000, K=13, L=20, n_out=7),
        "pooling_mixed_lengths": lambda s, d: _with_lengths(
            support.opsa_case(s, d, J=sum(MIXED_LENGTHS), K=5, L=40, n_out=len(MIXED_LENGTHS)), "indices_output", MIXED_LENGTHS
        ),
        "many_columns": lambda s, d: support.opsa_case(s, d, J=700, K=16, L=128, n_out=31, allow_empty=True),
        "ragged_columns": lambda s, d: support.opsa_case(s, d, J=500, K=20, L=70, n_out=23, allow_empty=True),
        # (rows of B that end inside a block of 64 or 32 columns whose lanes hold 4 or 2 consecutive ones)
        "columns_in_fours": lambda s, d: support.opsa_case(s, d, J=600, K=7, L=72, n_out=29, allow_empty=True),
        "columns_in_twos": lambda s, d: support.opsa_case(s, d, J=600, K=18, L=18, n_out=29, allow_empty=True),
    },
    "opsaw": {
        "tiny": lambda s, d: support.opsaw_case(s, d, E=6, K=2, L=3, n_nodes=4, allow_empty=True),
        "ragged": lambda s, d: support.opsaw_case(s, d, E=1000, K=13, L=32, n_nodes=37, allow_empty=True),
        "long_segments": lambda s, d: support.opsaw_case(s, d, E=3000, K=5, L=7, n_nodes=6),
        "hub_sender": lambda s, d: _hub(support.opsaw_case(s, d, E=2600, K=3, L=5, n_nodes=9), "indices_W"),
        "mostly_empty": lambda s, d: support.opsaw_case(s, d, E=20, K=4, L=4, n_nodes=300, allow_empty=True),
        "sparse_with_hubs": lambda s, d: _with_sender_counts(
            support.opsaw_case(s, d, E=6000, K=4, L=32, n_nodes=300, allow_empty=True), "indices_W", SENDER_COUNTS
        ),
        # (more than 4000 nodes: the senders' edges are listed in the order of arrival and sorted by their users)
        "many_nodes_with_hubs": lambda s, d: _with_sender_counts(
            support.opsaw_case(s, d, E=70000, K=4, L=24, n_nodes=4500, allow_empty=True), "indices_W", SENDER_COUNTS
        ),
        "forty_five_per_sender": lambda s, d: support.opsaw_case(s, d, E=4500, K=6, L=32, n_nodes=100),
        "sparse_tall": lambda s, d: support.opsaw_case(s, d, E=700, K=40, L=24, n_nodes=60, allow_empty=True),
        "sparse_taller": lambda s, d: support.opsaw_case(s, d, E=700, K=70, L=24, n_nodes=60, allow_empty=True),
        "fifty_seven_by_eighty": lambda s, d: support.opsaw_case(s, d, E=700, K=57, L=80, n_nodes=40, allow_empty=True),
        "pooling": lambda s, d: support.opsaw_case(s, d, E=5000, K=13, L=32, n_nodes=7),
        "pooling_mixed_lengths": lambda s, d: _with_lengths(
            support.opsaw_case(s, d, E=sum(MIXED_LENGTHS), K=3, L=17, n_nodes=len(MIXED_LENGTHS)), "indices_output", MIXED_LENGTHS
        ),
        "many_columns": lambda s, d: support.opsaw_case(s, d, E=700, K=32, L=192, n_nodes=31, allow_empty=True),
        "ragged_columns": lambda s, d: support.opsaw_case(s, d, E=500, K=9, L=131, n_nodes=23, allow_empty=True),
        "columns_in_fours": lambda s, d: support.opsaw_case(s, d, E=600, K=7, L=72, n_nodes=29, allow_empty=True),
        "columns_in_twos": lambda s, d: support.opsaw_case(s, d, E=600, K=18, L=18, n_nodes=29, allow_empty=True),
    },
    "sasaw": {
        "tiny": lambda s, d: support.sasaw_case(s, d, E=6, nA=2, L=3, n_nodes=4, n2=2, n3=2, N=5, allow_empty=True),
        "ragged": lambda s, d: support.sasaw_case(s, d, E=700, nA=9, L=32, n_nodes=29, n2=9, n3=9, N=250, allow_empty=True),
        "rectangular": lambda s, d: support.sasaw_case(s, d, E=300, nA=7, L=10, n_nodes=13, n2=5, n3=15, N=90, allow_empty=True),
        "hub_sender": lambda s, d: _hub(
            support.sasaw_case(s, d, E=2300, nA=3, L=4, n_nodes=7, n2=2, n3=3, N=10), "indices_W_1"
        ),
        "mostly_empty": lambda s, d: support.sasaw_case(s, d, E=15, nA=3, L=5, n_nodes=200, n2=3, n3=2, N=7, allow_empty=True),
        "sparse_with_hubs": lambda s, d: _with_sender_counts(
            support.sasaw_case(s, d, E=6000, nA=4, L=8, n_nodes=300, n2=3, n3=5, N=40, allow_empty=True),
            "indices_W_1", SENDER_COUNTS
        ),
        # (more than 4000 nodes: the senders' edges are listed in the order of arrival and sorted by their users)
        "many_nodes_with_hubs": lambda s, d: _with_sender_counts(
            support.sasaw_case(s, d, E=70000, nA=4, L=24, n_nodes=6500, n2=3, n3=5, N=40, allow_empty=True),
            "indices_W_1", SENDER_COUNTS
        ),
        "forty_five_per_sender": lambda s, d: support.sasaw_case(s, d, E=2250, nA=4, L=16, n_nodes=50, n2=4, n3=3, N=30),
        # (48 to 64 edges per sender on average: too many for the slots, listed by arrival)
        "sixty_per_sender": lambda s, d: support.sasaw_case(s, d, E=3000, nA=4, L=16, n_nodes=50, n2=4, n3=3, N=30),
        "many_columns": lambda s, d: support.sasaw_case(s, d, E=500, nA=9, L=128, n_nodes=21, n2=9, n3=9, N=120, allow_empty=True),
        "ragged_columns": lambda s, d: support.sasaw_case(s, d, E=400, nA=4, L=70, n_nodes=17, n2=6, n3=11, N=80, allow_empty=True),
        "three_blocks": lambda s, d: support.sasaw_case(s, d, E=300, nA=16, L=164, n_nodes=40, n2=16, n3=16, N=300, allow_empty=True),
        # more than 16 values of a component index: the forward pass takes the index ranges in parts.
        # The shape of the reference's own benchmark (mops/benchmarks/sasaw.cpp:10-51: 13 x 7 x 100
        # components, 900 entries, 60 edges per node), and 25 components each (spherical harmonics up to l = 4)
        "hundred_output_rows": lambda s, d: support.sasaw_case(s, d, E=3000, nA=13, L=32, n_nodes=50, n2=7, n3=100, N=900),
        "twenty_five_components": lambda s, d: support.sasaw_case(s, d, E=1500, nA=25, L=32, n_nodes=60, n2=25, n3=25, N=2000, allow_empty=True),
        "ragged_parts": lambda s, d: support.sasaw_case(s, d, E=700, nA=17, L=20, n_nodes=31, n2=33, n3=40, N=700, allow_empty=True),
    },
}  # fmt: skip


# Large and lopsided inputs: many times the BASELINE sizes, one receiver that
# owns almost every edge, senders named by tens of thousands of edges, feature
# counts beyond the matrix-core paths (the general kernels).
LARGE = {
    "hpe": {
        "many_rows": lambda s, d: support.hpe_case(s, d, I=300000, nA=40, J=300, K=4),
        "many_monomials": lambda s, d: support.hpe_case(s, d, I=500, nA=60, J=40000, K=5),
        "many_rows_long_table": lambda s, d: support.hpe_case(s, d, I=5000, nA=30, J=6000, K=3),
        "many_rows_order1": lambda s, d: support.hpe_case(s, d, I=4100, nA=7, J=50, K=1),
        "many_rows_very_long_table": lambda s, d: support.hpe_case(s, d, I=4096, nA=20, J=45000, K=3),
    },
    "sap": {
        "many_rows": lambda s, d: support.sap_case(s, d, I=1000003, nA=13, nB=7, K=900, nO=20),
        # (enough rows for the forward kernel whose wavefronts walk over tiles, too few for the vjp's in float32)
        "rows_between": lambda s, d: support.sap_case(s, d, I=150001, nA=13, nB=7, K=900, nO=20),
        "long_table": lambda s, d: support.sap_case(s, d, I=20000, nA=16, nB=16, K=6000, nO=30),
        "big_table_dimensions": lambda s, d: support.sap_case(s, d, I=5000, nA=40, nB=30, K=3000, nO=50),
        "tiles_beyond_64k": lambda s, d: support.sap_case(s, d, I=2000, nA=40, nB=40, K=3000, nO=60),
    },
    "opsa": {
        "many_edges": lambda s, d: support.opsa_case(s, d, J=1000003, K=13, L=20, n_out=30000, allow_empty=True),
        "one_receiver": lambda s, d: _one_receiver(support.opsa_case(s, d, J=120000, K=13, L=20, n_out=50), "indices_output"),
        "wide_rows": lambda s, d: support.opsa_case(s, d, J=20000, K=50, L=200, n_out=300, allow_empty=True),
        # (more than 64 columns of A and rows of grad_output beyond 64 KB: the vjp that keeps them in global memory)
        "tall_wide_rows": lambda s, d: support.opsa_case(s, d, J=8000, K=70, L=300, n_out=100, allow_empty=True),
    },
    "opsaw": {
        "many_edges": lambda s, d: support.opsaw_case(s, d, E=500001, K=16, L=64, n_nodes=20000, allow_empty=True),
        "one_receiver_one_sender": lambda s, d: _hub(
            _one_receiver(support.opsaw_case(s, d, E=120000, K=13, L=32, n_nodes=50), "indices_output"), "indices_W"
        ),
        "wide_rows": lambda s, d: support.opsaw_case(s, d, E=20000, K=40, L=300, n_nodes=300, allow_empty=True),
        "tall_wide_rows": lambda s, d: support.opsaw_case(s, d, E=8000, K=70, L=300, n_nodes=100, allow_empty=True),
    },
    "sasaw": {
        "many_edges": lambda s, d: support.sasaw_case(s, d, E=300001, nA=9, L=32, n_nodes=10000, allow_empty=True),
        "one_receiver_one_sender": lambda s, d: _hub(
            _one_receiver(support.sasaw_case(s, d, E=60000, nA=9, L=32, n_nodes=40), "indices_output_1"), "indices_W_1"
        ),
        "sixteen": lambda s, d: support.sasaw_case(s, d, E=30000, nA=16, L=64, n_nodes=900, n2=16, n3=16, N=700),
        # (a hundred edges per node on a graph too large for every workgroup to read the whole sender index: the
        # edges put in the order of their senders by a counting sort, grad_W by the forward kernel of sasaw_mfma.hip)
        "dense_large_graph": lambda s, d: support.sasaw_case(s, d, E=400000, nA=4, L=16, n_nodes=4000, n2=3, n3=4, N=30),
        "beyond_the_matrix_path": lambda s, d: support.sasaw_case(
            s, d, E=8000, nA=20, L=100, n_nodes=300, n2=18, n3=25, N=900, allow_empty=True
        ),
    },
}  # fmt: skip


def _one_receiver(case, key):
    """Nine edges in ten go to output row 3 (the index stays sorted)."""
    index = case[key]
    index[len(index) // 20 : len(index) * 19 // 20] = 3
    case[key] = np.sort(index)
    return case


def _with_lengths(case, key, lengths):
    """Scatter index with exactly these segment lengths (row r gets lengths[r] edges)."""
    index = np.repeat(np.arange(len(lengths)), lengths).astype(np.int32)
    assert len(index) == len(case[key])
    case[key] = index
    return case


# lengths around the distance at which long segments are cut (256), rows without edges, one row over many cuts
MIXED_LENGTHS = [0, 1700, 3, 0, 2300, 255, 256, 257, 512, 1, 0, 1900, 0, 769]


# senders of a sparse graph (20 edges per sender on average) named by exactly this many edges:
# around the 64 edges one wavefront holds, around the 128 places a sender owns, and far beyond
SENDER_COUNTS = {5: 1000, 7: 128, 9: 129, 11: 64, 13: 65, 15: 0, 299: 127}


def _with_sender_counts(case, key, counts):
    """Sender index in which sender v is named by exactly counts[v] edges, at random positions."""
    index = case[key]
    n_nodes = int(index.max()) + 1
    for value in counts:
        index[index == value] = (value + 1) % n_nodes
    assert not set(counts) & {(value + 1) % n_nodes for value in counts}
    positions = np.random.default_rng(len(index)).permutation(len(index))
    used = 0
    for value, count in counts.items():
        index[positions[used : used + count]] = value
        used += count
    for value, count in counts.items():
        assert int((index == value).sum()) == count
    return case


def _hub(case, key):
    """Most edges name the same sender: one gather list longer than the LDS sort buffer."""
    case[key][: len(case[key]) * 3 // 4] = 2
    return case


ALL = [(op, name) for op, cases in CASES.items() for name in cases]


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f64"])
@pytest.mark.parametrize("op,name", ALL)
def test_forward(oracle, device, op, name, dtype):
    case = CASES[op][name](101, dtype)
    expected = cpu_forward(oracle, op, case)
    actual = hip_forward(op, to_device(case, device)).cpu().numpy()
    assert_close(actual, expected, dtype, f"{op}/{name}")
    # also against the dense float64 formulation, which shares nothing with the oracle
    assert_close(actual, OPS[op].dense(case), dtype, f"{op}/{name} dense")


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f64"])
@pytest.mark.parametrize("op,name", [(op, name) for op, name in ALL if op in ("opsa", "opsaw")])
def test_forward_with_64_bit_offsets(oracle, device, monkeypatch, op, name, dtype):
    """The forward kernels for tensors of 4 GB and more, forced onto small inputs."""
    case = CASES[op][name](101, dtype)
    on_device = to_device(case, device)
    narrow = hip_forward(op, on_device).cpu().numpy()
    monkeypatch.setenv("MOPS_AMD_WIDE_OFFSETS", "1")
    wide = hip_forward(op, on_device).cpu().numpy()
    assert_close(wide, cpu_forward(oracle, op, case), dtype, f"{op}/{name} wide")
    # same sums in the same order on both paths
    assert np.array_equal(wide, narrow), f"{op}/{name}"


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f64"])
@pytest.mark.parametrize("op,name", ALL)
def test_vjp(oracle, device, op, name, dtype):
    case = CASES[op][name](202, dtype)
    expected = cpu_vjp(oracle, op, case)
    actual = hip_vjp(op, to_device(case, device))
    for key in OPS[op].differentiable:
        assert_close(actual[key].cpu().numpy(), expected[key], dtype, f"{op}/{name} grad_{key}")


@pytest.mark.parametrize("shift", [1, 2, 3])
@pytest.mark.parametrize("op,key", [("opsaw", "indices_W"), ("sasaw", "indices_W_1")])
def test_sender_index_off_the_vector_boundary(oracle, device, op, key, shift):
    """The sender index starts 4, 8 or 12 bytes after a 16-byte boundary: the kernels that read
    it 128 bits at a time must take their other way, with the same results."""
    import torch

    for name in ("ragged", "sparse_with_hubs"):
        case = CASES[op][name](707, np.float32)
        expected = cpu_vjp(oracle, op, case)
        on_device = to_device(case, device)
        index = on_device[key]
        longer = torch.zeros(len(index) + 8, dtype=index.dtype, device=index.device)
        base = (-longer.data_ptr() // 4) % 4  # elements up to the next 16-byte boundary
        view = longer[base + shift : base + shift + len(index)]
        view.copy_(index)
        assert view.data_ptr() % 16 == 4 * shift
        on_device[key] = view
        actual = hip_vjp(op, on_device)
        for gradient in OPS[op].differentiable:
            assert_close(actual[gradient].cpu().numpy(), expected[gradient], np.float32, f"{op}/{name} grad_{gradient}")


@pytest.mark.parametrize("op", list(OPS))
def test_vjp_subsets_of_gradients(oracle, device, op):
    """Every subset of requested gradients gives the same values as all of them."""
    case = CASES[op]["ragged"](303, np.float64)
    on_device = to_device(case, device)
    full = hip_vjp(op, on_device)
    names = OPS[op].differentiable
    for r in range(len(names)):
        for wanted in itertools.combinations(names, r):
            partial = hip_vjp(op, on_device, wanted=list(wanted))
            for key in names:
                if key in wanted:
                    assert np.array_equal(partial[key].cpu().numpy(), full[key].cpu().numpy()), (op, wanted, key)
                else:
                    assert partial[key] is None


def test_sasaw_in_parts_subsets_of_gradients(device):
    """The same where the index ranges are taken in parts (launches that add to each other's results)."""
    case = CASES["sasaw"]["ragged_parts"](304, np.float64)
    on_device = to_device(case, device)
    full = hip_vjp("sasaw", on_device)
    for wanted in (["A"], ["B"], ["W"], ["A", "W"], ["B", "W"]):
        partial = hip_vjp("sasaw", on_device, wanted=wanted)
        for key in ("A", "B", "W"):
            if key in wanted:
                assert np.array_equal(partial[key].cpu().numpy(), full[key].cpu().numpy()), (wanted, key)
            else:
                assert partial[key] is None


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f64"])
def test_sap_many_rows_subsets_of_gradients(device, dtype):
    """The same for the SAP kernels whose wavefronts walk over the rows (300 000 rows and more)."""
    case = support.sap_case(305, dtype, I=300011, nA=13, nB=7, K=900, nO=20)
    on_device = to_device(case, device)
    full = hip_vjp("sap", on_device)
    for wanted in (["A"], ["B"]):
        partial = hip_vjp("sap", on_device, wanted=wanted)
        for key in ("A", "B"):
            if key in wanted:
                assert np.array_equal(partial[key].cpu().numpy(), full[key].cpu().numpy()), (wanted, key)
            else:
                assert partial[key] is None


@pytest.mark.parametrize("op", ["opsa", "opsaw", "sasaw"])
def test_rows_without_edges_are_exactly_zero(device, op):
    case = CASES[op]["ragged"](404, np.float32)
    key = "indices_output_1" if op == "sasaw" else "indices_output"
    index = case[key]
    index[index == 1] = 2
    case[key] = np.sort(index)
    out = hip_forward(op, to_device(case, device)).cpu().numpy()
    assert np.all(out[1] == 0.0)
    assert not np.any(np.isnan(out))


def test_no_edges_at_all(device):
    """Zero input rows: outputs are all zero, gradients are empty. (Also for many nodes: the
    ways of listing the senders' edges that large graphs take need edges to list.)"""
    for op, name in (("opsa", "tiny"), ("opsaw", "tiny"), ("sasaw", "tiny"), ("opsaw", "many_nodes_with_hubs"), ("sasaw", "many_nodes_with_hubs")):
        case = CASES[op][name](1, np.float64)
        for key in ("A", "B"):
            case[key] = case[key][:0]
        for key in ("indices_output", "indices_W", "indices_output_1", "indices_W_1"):
            if key in case:
                case[key] = case[key][:0]
        out = hip_forward(op, to_device(case, device)).cpu().numpy()
        assert out.size > 0 and np.all(out == 0.0)
        grads = hip_vjp(op, to_device(case, device))
        assert grads["A"].numel() == 0 and grads["B"].numel() == 0
        if "W" in grads:
            assert np.all(grads["W"].cpu().numpy() == 0.0)


@pytest.mark.parametrize("op", list(OPS))
def test_bit_reproducible(device, op):
    """No atomics on floating-point data: two runs give identical bits."""
    case = to_device(CASES[op]["ragged"](505, np.float32), device)
    first = hip_forward(op, case).cpu().numpy()
    second = hip_forward(op, case).cpu().numpy()
    assert np.array_equal(first, second)
    g1 = hip_vjp(op, case)
    g2 = hip_vjp(op, case)
    for key in OPS[op].differentiable:
        assert np.array_equal(g1[key].cpu().numpy(), g2[key].cpu().numpy()), (op, key)


ALL_LARGE = [(op, name) for op, cases in LARGE.items() for name in cases]


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f64"])
@pytest.mark.parametrize("op,name", ALL_LARGE)
def test_large_inputs(oracle, device, op, name, dtype):
    case = LARGE[op][name](808, dtype)
    on_device = to_device(case, device)
    # Expected values from the oracle in float64 on the same (already rounded) inputs; the bar is
    # the north star's unless the sum is measured to be ill-conditioned (support.calibrated_bar:
    # the float32 oracle's own distance from the float64 result, the ratio of the terms'
    # magnitudes to the result in float64), and says so when it is.
    exact = support.in_float64(case)
    absolute = support.magnitudes(case)
    single = dtype == np.float32

    def check(actual, expected, same_dtype, sums, what):
        error, bar, reason = support.assert_calibrated(actual, expected, dtype, what, same_dtype, sums)
        if bar != support.TOLERANCE[np.dtype(dtype)]:
            print(f"{what}: error {error:.2e}, bar {bar:.2e}: {reason}", flush=True)

    actual = hip_forward(op, on_device).cpu().numpy()
    check(
        actual, cpu_forward(oracle, op, exact), cpu_forward(oracle, op, case) if single else None,
        None if single else cpu_forward(oracle, op, absolute), f"{op}/{name} forward",
    )  # fmt: skip
    expected = cpu_vjp(oracle, op, exact)
    same = cpu_vjp(oracle, op, case) if single else {}
    sums = {} if single else cpu_vjp(oracle, op, absolute)
    gradients = hip_vjp(op, on_device)
    for key in OPS[op].differentiable:
        check(gradients[key].cpu().numpy(), expected[key], same.get(key), sums.get(key), f"{op}/{name} grad_{key}")


# ---- pointers that are aligned to an element and no more -------------------
OFF_BOUNDARY = {
    "hpe": lambda d: support.hpe_case(31, d, I=300, nA=20, J=150, K=3),
    "sap": lambda d: support.sap_case(32, d, I=700, nA=13, nB=7, K=300, nO=20),
    "opsa": lambda d: support.opsa_case(33, d, J=3000, K=13, L=20, n_out=90, allow_empty=True),
    "opsa_wide": lambda d: support.opsa_case(34, d, J=2000, K=20, L=64, n_out=60, allow_empty=True),
    "opsaw": lambda d: support.opsaw_case(35, d, E=3000, K=13, L=32, n_nodes=90, allow_empty=True),
    "opsaw_many_senders": lambda d: support.opsaw_case(36, d, E=20000, K=4, L=16, n_nodes=5000, allow_empty=True),
    "sasaw": lambda d: support.sasaw_case(37, d, E=3000, nA=9, L=32, n_nodes=90, allow_empty=True),
    "sasaw_parts": lambda d: support.sasaw_case(38, d, E=900, nA=17, L=20, n_nodes=31, n2=20, n3=18, N=500, allow_empty=True),
}


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f64"])
@pytest.mark.parametrize("name", list(OFF_BOUNDARY))
def test_pointers_one_element_off_the_vector_boundaries(oracle, device, name, dtype):
    """Every tensor (inputs, indices, outputs) starts one element behind a 256-byte boundary, so no
    pointer is aligned to 8 or 16 bytes: the kernels that move 8 or 16 bytes per lane must step aside
    for the ones that move single elements."""
    import torch

    from mops_amd._c_lib import device_library

    op = name.split("_")[0]
    spec = OPS[op]
    case = OFF_BOUNDARY[name](dtype)

    def shifted(tensor):
        room = torch.empty(tensor.numel() + 1, dtype=tensor.dtype, device=device)
        view = room[1:].view(tensor.shape)
        view.copy_(tensor)
        assert view.data_ptr() % 256 == tensor.element_size()
        return view

    on_device = {
        key: shifted(value) if isinstance(value, torch.Tensor) else value
        for key, value in to_device(case, device).items()
    }
    library = device_library()
    support._bind_stream(library, device)
    inputs = [on_device[key] for key in spec.inputs]
    output = shifted(torch.full(spec.output_shape(on_device), float("nan"), dtype=on_device["A"].dtype, device=device))
    library.call(spec.function, output, *inputs)
    assert_close(output.cpu().numpy(), cpu_forward(oracle, op, case), dtype, f"{name} forward")
    gradients = [shifted(torch.full_like(on_device[key], float("nan"))) for key in spec.differentiable]
    library.call(spec.function + "_vjp", *gradients, on_device["grad_output"], *inputs)
    expected = cpu_vjp(oracle, op, case)
    for key, got in zip(spec.differentiable, gradients):
        assert_close(got.cpu().numpy(), expected[key], dtype, f"{name} grad_{key}")


# ---- inputs that are not finite ---------------------------------------------
NON_FINITE = [
    # operation, tensor and element that is set, how many rows of each result may differ from the oracle in
    # where they are finite (the kernels multiply through dense tables and through groups of 16 edges: a
    # zero times an infinity or a NaN is a NaN, where the reference never forms the product)
    ("sap", lambda d: support.sap_case(61, d, I=2000), "A", (5, 3), 1),
    ("opsa", lambda d: support.opsa_case(62, d, J=6000, n_out=200), "grad_output", (7, 2, 3), 32),
    ("opsa", lambda d: support.opsa_case(63, d, J=6000, n_out=200), "B", (100, 3), 1),
    ("opsaw", lambda d: support.opsaw_case(64, d, E=6000, n_nodes=200), "W", (9, 3), 64),
    ("sasaw", lambda d: support.sasaw_case(65, d, E=6000, n_nodes=200), "A", (100, 3), 64),
    ("sasaw", lambda d: support.sasaw_case(66, d, E=6000, n_nodes=200), "grad_output", (7, 2, 3), 64),
    ("hpe", lambda d: support.hpe_case(67, d, I=100), "A", (5, 3), 0),
]


@pytest.mark.parametrize("value", [float("nan"), float("inf")], ids=["nan", "inf"])
@pytest.mark.parametrize("op,build,tensor,element,rows", NON_FINITE, ids=[f"{o}-{t}" for o, _, t, _, _ in NON_FINITE])
def test_an_input_that_is_not_finite(oracle, device, op, build, tensor, element, rows, value):
    """Where the oracle's result is not finite, so is the device's; where both are finite they agree;
    the device may have a NaN where the oracle has a number only in a bounded number of rows around the
    element (documented deviation: dense tables and groups of 16 edges)."""
    dtype = np.float64 if op == "hpe" else np.float32
    case = build(dtype)
    case[tensor][element] = value
    on_device = to_device(case, device)
    results = [("forward", hip_forward(op, on_device).cpu().numpy(), cpu_forward(oracle, op, case))]
    expected = cpu_vjp(oracle, op, case)
    for key, got in hip_vjp(op, on_device).items():
        results.append((f"grad_{key}", got.cpu().numpy(), expected[key]))
    for name, got, want in results:
        bad_got, bad_want = ~np.isfinite(got), ~np.isfinite(want)
        assert not np.any(bad_want & ~bad_got), (op, name, "finite where the oracle is not")
        extra = bad_got & ~bad_want
        extra_rows = np.unique(np.nonzero(extra.reshape(extra.shape[0], -1))[0]).size
        assert extra_rows <= rows, (op, name, extra_rows)
        both = ~bad_got & ~bad_want
        assert_close(np.where(both, got, 0), np.where(both, want, 0), dtype, f"{op} {name} beside the {value}")


# ---- BASELINE configurations at full size ---------------------------------
BASELINE = [
    ("hpe", 0, np.float64, lambda d: support.hpe_case(0, d)),
    ("sap", 1, np.float32, lambda d: support.sap_case(1, d)),
    ("sap", 1, np.float64, lambda d: support.sap_case(1, d)),
    ("opsa", 2, np.float32, lambda d: support.opsa_case(2, d)),
    ("opsa", 2, np.float64, lambda d: support.opsa_case(2, d)),
    ("opsaw", 3, np.float32, lambda d: support.opsaw_case(3, d)),
    ("sasaw", 4, np.float32, lambda d: support.sasaw_case(4, d)),
    ("sasaw", 4, np.float64, lambda d: support.sasaw_case(4, d)),
]


@pytest.mark.parametrize(
    "op,config,dtype,build", BASELINE, ids=[f"c{c}-{o}-{np.dtype(t).name}" for o, c, t, _ in BASELINE]
)
def test_baseline_configuration(oracle, device, op, config, dtype, build):
    case = build(dtype)
    on_device = to_device(case, device)
    out = hip_forward(op, on_device).cpu().numpy()
    assert_close(out, cpu_forward(oracle, op, case), dtype, f"c{config} {op} forward")
    expected = cpu_vjp(oracle, op, case)
    grads = hip_vjp(op, on_device)
    for key in OPS[op].differentiable:
        assert_close(grads[key].cpu().numpy(), expected[key], dtype, f"c{config} {op} grad_{key}")

    # size-independent properties, float64 accumulation on the host
    rng = np.random.default_rng(99)
    g = case["grad_output"].astype(np.float64)
    if op != "hpe":
        # adjoint identity: <vjp_x(g), dx> == <g, f(x := dx)> (multilinear operations)
        for key in OPS[op].differentiable:
            dx = rng.normal(size=case[key].shape).astype(dtype)
            swapped = dict(on_device)
            swapped[key] = to_device({"x": dx}, device)["x"]
            right = np.sum(g * hip_forward(op, swapped).cpu().numpy())
            product = grads[key].cpu().numpy().astype(np.float64) * dx
            left = np.sum(product)
            assert abs(left - right) <= support.TOLERANCE[np.dtype(dtype)] * 100 * np.sum(np.abs(product)), (op, key)
    else:
        # homogeneity: scaling A by t scales O by t^order
        scaled = dict(on_device)
        scaled["A"] = on_device["A"] * 2.0
        order = case["indices_A"].shape[1]
        assert_close(hip_forward(op, scaled).cpu().numpy(), out * 2.0**order, dtype, "hpe homogeneity")


# ---- second order: vjp_vjp of HPE, SAP, OPSA -------------------------------
SECOND = [(op, name) for op in support.SECOND_ORDER for name in CASES[op]]


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f64"])
@pytest.mark.parametrize("op,name", SECOND)
def test_vjp_vjp(oracle, device, op, name, dtype):
    case = support.add_cotangents(CASES[op][name](606, dtype), op)
    # (second-order results are sums over the first-order ones: the bar is calibrated like that of
    # the large inputs, support.calibrated_bar)
    expected = support.cpu_vjp_vjp(oracle, op, support.in_float64(case))
    single = dtype == np.float32
    same = support.cpu_vjp_vjp(oracle, op, case) if single else {}
    sums = {} if single else support.cpu_vjp_vjp(oracle, op, support.magnitudes(case))
    actual = support.hip_vjp_vjp(op, to_device(case, device))
    for key in ["grad_output"] + OPS[op].differentiable:
        support.assert_calibrated(
            actual[key].cpu().numpy(), expected[key], dtype, f"{op}/{name} second order {key}", same.get(key), sums.get(key)
        )


@pytest.mark.parametrize("op", support.SECOND_ORDER)
def test_vjp_vjp_absent_cotangents_and_skipped_outputs(oracle, device, op):
    case = support.add_cotangents(CASES[op]["ragged"](707, np.float64), op)
    on_device = to_device(case, device)
    names = OPS[op].differentiable
    outputs = ["grad_output"] + names
    full = {k: v.cpu().numpy() for k, v in support.hip_vjp_vjp(op, on_device).items()}
    for r in range(len(names) + 1):
        for have in itertools.combinations(names, r):
            expected = support.cpu_vjp_vjp(oracle, op, case, have=list(have))
            actual = support.hip_vjp_vjp(op, on_device, have=list(have))
            for key in outputs:
                assert_close(actual[key].cpu().numpy(), expected[key], np.float64, f"{op} have={have} {key}")
    for alone in outputs:
        actual = support.hip_vjp_vjp(op, on_device, wanted=[alone])
        assert np.array_equal(actual[alone].cpu().numpy(), full[alone]), (op, alone)
        assert all(value is None for key, value in actual.items() if key != alone)


@pytest.mark.parametrize("op,config,dtype,build", [b for b in BASELINE if b[0] in support.SECOND_ORDER],
                         ids=[f"c{c}-{o}-{np.dtype(t).name}" for o, c, t, _ in BASELINE if o in support.SECOND_ORDER])
def test_vjp_vjp_baseline_configuration(oracle, device, op, config, dtype, build):
    case = support.add_cotangents(build(dtype), op)
    on_device = to_device(case, device)
    expected = support.cpu_vjp_vjp(oracle, op, case)
    actual = support.hip_vjp_vjp(op, on_device)
    for key in ["grad_output"] + OPS[op].differentiable:
        assert_close(actual[key].cpu().numpy(), expected[key], dtype, f"c{config} {op} second order {key}")
    # size-independent property: the second-order function is the transpose of the
    # derivative of the vjp, so <gg, vjp(g + dg) - vjp(g)> == <grad_grad_output, dg> exactly
    # (the vjp is linear in grad_output)
    rng = np.random.default_rng(17)
    dg = rng.normal(size=case["grad_output"].shape).astype(dtype)
    shifted = dict(on_device)
    shifted["grad_output"] = to_device({"x": dg}, device)["x"]
    moved = hip_vjp(op, shifted)
    left = sum(
        np.sum(case["grad_grad_" + key].astype(np.float64) * moved[key].cpu().numpy())
        for key in OPS[op].differentiable
    )
    product = actual["grad_output"].cpu().numpy().astype(np.float64) * dg
    assert abs(left - np.sum(product)) <= support.TOLERANCE[np.dtype(dtype)] * 100 * np.sum(np.abs(product)), op


# ---- scatter index in any order (host semantics on the device) -------------
@pytest.fixture
def unsorted_accepted(device):
    import mops_amd

    previous = mops_amd.accept_unsorted_indices(True)
    yield
    mops_amd.accept_unsorted_indices(previous)


def _shuffled(case, op, seed):
    """The same edges in a random order (so the scatter index is no longer sorted)."""
    rng = np.random.default_rng(seed)
    per_edge = {
        "opsa": ["A", "B", "indices_output"],
        "opsaw": ["A", "B", "indices_W", "indices_output"],
        "sasaw": ["A", "B", "indices_W_1", "indices_output_1"],
    }[op]
    order = rng.permutation(case["A"].shape[0])
    for key in per_edge:
        case[key] = np.ascontiguousarray(case[key][order])
    return case


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f64"])
@pytest.mark.parametrize("op", ["opsa", "opsaw", "sasaw"])
@pytest.mark.parametrize("name", ["ragged", "long_segments", "mostly_empty"])
def test_unsorted_scatter_index(oracle, device, unsorted_accepted, op, name, dtype):
    if name not in CASES[op]:
        pytest.skip("no such case for this operation")
    case = _shuffled(CASES[op][name](909, dtype), op, 5)
    key = "indices_output_1" if op == "sasaw" else "indices_output"
    assert np.any(np.diff(case[key]) < 0)
    on_device = to_device(case, device)
    actual = hip_forward(op, on_device).cpu().numpy()
    assert_close(actual, cpu_forward(oracle, op, case), dtype, f"{op}/{name} unsorted forward")
    expected = cpu_vjp(oracle, op, case)
    gradients = hip_vjp(op, on_device)
    for name_ in OPS[op].differentiable:
        assert_close(gradients[name_].cpu().numpy(), expected[name_], dtype, f"{op}/{name} unsorted grad_{name_}")
    # only some of the gradients
    partial = hip_vjp(op, on_device, wanted=["B"])
    assert np.array_equal(partial["B"].cpu().numpy(), gradients["B"].cpu().numpy())
    if op in support.SECOND_ORDER:
        support.add_cotangents(case, op)
        on_device = to_device(case, device)
        second = support.hip_vjp_vjp(op, on_device)
        expected = support.cpu_vjp_vjp(oracle, op, case)
        for name_ in ["grad_output"] + OPS[op].differentiable:
            assert_close(second[name_].cpu().numpy(), expected[name_], dtype, f"{op}/{name} unsorted second {name_}")


def test_sorted_index_takes_the_usual_path_when_unsorted_is_accepted(device, unsorted_accepted):
    """With the switch on, a sorted index gives the same bits as with the switch off."""
    import mops_amd

    case = to_device(CASES["opsaw"]["ragged"](111, np.float32), device)
    with_switch = hip_forward("opsaw", case).cpu().numpy()
    mops_amd.accept_unsorted_indices(False)
    without = hip_forward("opsaw", case).cpu().numpy()
    mops_amd.accept_unsorted_indices(True)
    assert np.array_equal(with_switch, without)
