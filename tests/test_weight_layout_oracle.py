"""Pins of oracle/weight_layout_oracle.py: the byte permutation the reference's compiler applies
to the constant weight of a weight-only GEMM (R tao_compiler/mlir/disc/transforms/
disc_transform_weight_data_layout_for_weight_only_gemm.cc:54-300, composed at :362-370)."""
import numpy as np
import pytest

from oracle import weight_layout_oracle as L

SHAPES = [(64, 4), (64, 128), (128, 8), (192, 20), (1280, 200), (1024, 1024)]


@pytest.mark.parametrize("k,n", SHAPES)
def test_every_step_and_the_composition_are_permutations(k, n):
    idx = np.arange(k * n, dtype=np.int64).reshape(k, n)
    steps = [L.permute_b_rows(idx), L.subbyte_transpose(idx),
             L.interleave_column_major(np.ascontiguousarray(idx.T)),
             L.add_bias_and_interleave_int8s(idx.reshape(-1)), L.forward(idx)]
    for out in steps:
        assert np.array_equal(np.sort(out.reshape(-1)), np.arange(k * n))


@pytest.mark.parametrize("k,n", SHAPES)
def test_inverse_of_forward_is_the_weight(k, n):
    w = np.random.default_rng(k + n).integers(0, 256, (k, n), dtype=np.uint8)
    f = L.forward(w)
    assert f.shape == (k, n) and f.dtype == np.uint8
    assert np.array_equal(L.inverse(f), w)
    assert not np.array_equal(f, w)


@pytest.mark.parametrize("k,n", [(64, 4), (64, 12), (128, 8), (192, 20)])
def test_array_form_equals_the_reference_loops(k, n):
    w = np.random.default_rng(7 * k + n).integers(0, 256, (k, n), dtype=np.uint8)
    assert np.array_equal(L.forward_loops(w), L.forward(w))


@pytest.mark.parametrize("k,n", SHAPES)
def test_closed_form_equals_the_composition(k, n):
    w = np.random.default_rng(3 * k + n).integers(0, 256, (k, n), dtype=np.uint8)
    assert np.array_equal(L.forward_closed_form(w), L.forward(w))


def test_positions_worked_out_by_hand():
    """K = 64, N = 4; pos = flat index k*4 + n of the source byte.
    Step 1 leaves P[r] = W[read(r)], read = 0,1,8,9,2,3,10,11,4,5,12,13,6,7,14,15 per 16 rows;
    step 2 T[n][r] = P[r][n]; step 3 puts column n's 64 bytes at (n/2)*128 + (n%2)*64; step 4
    swaps bytes 1 and 2 of each word.  So the result starts with column 0's rows
    read(0), read(2), read(1), read(3), read(4), read(6), ... = W rows 0, 8, 1, 9, 2, 10, ..."""
    k, n = 64, 4
    pos = L.forward_positions(k, n)
    rows = lambda a: [int(p) // n for p in a]          # noqa: E731
    cols = lambda a: [int(p) % n for p in a]           # noqa: E731
    assert rows(pos[:8]) == [0, 8, 1, 9, 2, 10, 3, 11] and cols(pos[:8]) == [0] * 8
    assert rows(pos[8:16]) == [4, 12, 5, 13, 6, 14, 7, 15]
    assert rows(pos[16:20]) == [16, 24, 17, 25]                       # the next block of 16 rows
    assert cols(pos[64:68]) == [1] * 4 and rows(pos[64:68]) == [0, 8, 1, 9]   # column 1 follows
    assert cols(pos[128:132]) == [2] * 4 and cols(pos[192:196]) == [3] * 4
    # K = 128: a column pair alternates in tiles of 64 rows
    pos = L.forward_positions(128, 4)
    assert cols(pos[0:256:64]) == [0, 1, 0, 1] and rows(pos[0:256:64]) == [0, 0, 64, 64]


@pytest.mark.parametrize("k,n", [(3, 5), (96, 8), (64, 6), (0, 4)])
def test_shapes_outside_the_pass_domain_are_refused(k, n):
    with pytest.raises(ValueError):
        L.forward(np.zeros((k, n), np.uint8))
