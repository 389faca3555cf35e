"""CPU restatement of the byte permutation the reference's compiler applies to the constant
weight of a weight-only quantized GEMM.

TEST INFRASTRUCTURE ONLY -- the checker for the runtime's inverse re-layout.  Nothing in the
shipped GPU path imports it.

The pass (R tao_compiler/mlir/disc/transforms/
disc_transform_weight_data_layout_for_weight_only_gemm.cc:305-410, run unconditionally from
R tao_compiler/mlir/disc/disc_compiler.cc:257-258) rewrites every `ral_pdll_weight_only_qgemm`
whose weight operand is a rank-2 `ui8` constant of shape [K, N]: it runs four functions over the
bytes (:362-370) and sets `weight_should_be_reordered = false`.  The four functions are restated
here one by one, each on arrays of "32-bit words" (groups of four consecutive bytes) exactly as
the reference reads them, but generic in the element type, so that the same code permutes an
array of byte *positions* and thereby yields the permutation itself.

The reference reads and writes outside its buffers unless K % 64 == 0 and N % 4 == 0
(`permute_B_rows_for_mixed_gemm` walks rows in blocks of 16 and columns as whole words; the
transpose stores 32-byte vectors guarded only by their first byte; the interleave maps a partial
64-row tile beyond its column pair), so only those shapes are defined and `check_shape` refuses
the others.

Pins (tests/test_weight_layout_oracle.py): every step and the composition are permutations; a
literal loop form (`forward_loops`) against the array form; a closed form of the composition
derived by hand from the four definitions (`forward_closed_form`); byte positions worked out on
paper.  The reference holds no expected bytes for this pass (its FileCheck test,
R tao_compiler/mlir/disc/transforms/tests/disc-convert-weight-layout-for-weight-only-gemm.mlir,
uses an all-zero weight and checks only the attribute).
"""
import numpy as np


def check_shape(k, n):
    if k <= 0 or n <= 0 or k % 64 or n % 4:
        raise ValueError("the layout pass is a permutation only for K % 64 == 0 and N % 4 == 0 "
                         "(got K = %d, N = %d)" % (k, n))


def permute_b_rows(w):
    """`permute_B_rows_for_mixed_gemm` (:241-300) with 8-bit elements: rows in blocks of 16,
    row `t` of the result's block is row `8*((t%4)/2) + t%2 + 2*(t/4)` of the input's; whole
    32-bit words move, the column does not change."""
    k, n = w.shape
    check_shape(k, n)
    words = w.reshape(k, n // 4, 4)
    t = np.arange(k) % 16
    read_row = (np.arange(k) - t) + 8 * ((t % 4) // 2) + t % 2 + 2 * (t // 4)
    return words[read_row].reshape(k, n)


def subbyte_transpose(w):
    """`subbyte_transpose_impl<INT8_WEIGHT_ONLY>` (:123-239): a plain [K, N] -> [N, K]
    transpose done in 64 x 64 tiles."""
    return np.ascontiguousarray(w.T)


def interleave_column_major(t):
    """`interleave_column_major_tensor` (:73-121) with 8-bit elements: `t` is the transposed
    tensor, i.e. N columns of K contiguous bytes = K/4 words each.  Column pairs share an output
    column of 2·K/4 words: word `r` of column `c` goes to word `2·base + 16·(c % 2) + r % 16`
    of output column `c / 2`, `base` = start of r's tile of 16 words (64 rows)."""
    n, k = t.shape
    check_shape(k, n)
    nvr = k // 4                                     # num_vec_rows
    words = t.reshape(n, nvr, 4)
    out = np.empty((n // 2, 2 * nvr, 4), dtype=t.dtype)
    r = np.arange(nvr)
    base = (r // 16) * 16
    for parity in (0, 1):
        out[:, 2 * base + 16 * parity + r % 16, :] = words[parity::2]
    return out.reshape(n // 2, 2 * k)


def add_bias_and_interleave_int8s(flat):
    """`add_bias_and_interleave_int8s_inplace` (:54-71): despite its name only the swap of
    bytes 1 and 2 of every group of four."""
    g = flat.reshape(-1, 4).copy()
    g[:, [1, 2]] = g[:, [2, 1]]
    return g.reshape(flat.shape)


def forward(w_kn):
    """The pass's composition (:362-370) on a [K, N] array; returns the reordered bytes in the
    shape the compiler keeps for the constant, [K, N]."""
    w_kn = np.ascontiguousarray(w_kn)
    k, n = w_kn.shape
    check_shape(k, n)
    x = permute_b_rows(w_kn)
    x = subbyte_transpose(x)
    x = interleave_column_major(x)
    x = add_bias_and_interleave_int8s(x.reshape(-1))
    return x.reshape(k, n)


def forward_loops(w_kn):
    """The same composition written as the reference's loops, index for index (slow: for small
    shapes; the array forms above are checked against it)."""
    w_kn = np.ascontiguousarray(w_kn)
    k, n = w_kn.shape
    check_shape(k, n)
    dt = w_kn.dtype
    # permute_B_rows_for_mixed_gemm (:241-300): B_ROWS_PER_MMA = 16, ELTS_PER_REG = 4
    num_vec_cols = n // 4
    src = w_kn.reshape(k * num_vec_cols, 4)
    dst = np.empty_like(src)
    for base_row in range(0, k, 16):
        for tile_row in range(16):
            tile_read_row = 8 * ((tile_row % 4) // 2) + tile_row % 2 + 2 * (tile_row // 4)
            for col in range(num_vec_cols):
                dst[(base_row + tile_row) * num_vec_cols + col] = \
                    src[(base_row + tile_read_row) * num_vec_cols + col]
    # subbyte_transpose_impl<INT8_WEIGHT_ONLY> (:123-239)
    src = dst.reshape(k, n)
    dst = np.empty((n, k), dtype=dt)
    for row in range(k):
        for col in range(n):
            dst[col, row] = src[row, col]
    # interleave_column_major_tensor (:73-121): rows_per_tile = 64, interleave = 2
    num_vec_rows = k // 4
    vec_rows_per_tile = 16
    src = dst.reshape(n * num_vec_rows, 4)
    dst = np.empty_like(src)
    for read_col in range(n):
        write_col = read_col // 2
        for base_vec_row in range(0, num_vec_rows, vec_rows_per_tile):
            for vec_read_row in range(base_vec_row,
                                      min(num_vec_rows, base_vec_row + vec_rows_per_tile)):
                vec_write_row = (2 * base_vec_row + vec_rows_per_tile * (read_col % 2)
                                 + vec_read_row % vec_rows_per_tile)
                dst[write_col * num_vec_rows * 2 + vec_write_row] = \
                    src[read_col * num_vec_rows + vec_read_row]
    # add_bias_and_interleave_int8s_inplace (:54-71)
    out = dst.reshape(-1).copy()
    for base in range(0, k * n, 4):
        out[base + 1], out[base + 2] = out[base + 2], out[base + 1]
    return out.reshape(k, n)


def forward_positions(k, n):
    """pos[i] = flat position in the [K, N] input of the byte the pass puts at flat position i."""
    return forward(np.arange(k * n, dtype=np.int64).reshape(k, n)).reshape(-1)


def inverse(reordered_kn):
    """Undo `forward`: the [K, N] weight the compiler started from."""
    r = np.ascontiguousarray(reordered_kn)
    k, n = r.shape
    out = np.empty(k * n, dtype=r.dtype)
    out[forward_positions(k, n)] = r.reshape(-1)
    return out.reshape(k, n)


def forward_closed_form(w_kn):
    """The same permutation from its closed form, derived by hand from the four definitions and
    used by the GPU kernel: with W_nk = W^T, the 16 bytes W_nk[n, 16j : 16j+16] land in one
    16-byte group of the result, at byte offset
        (n/2)·2K + (16j / 64)·128 + (n % 2)·64 + (16j % 64),
    in the order k-offsets 0,8,1,9,2,10,...,7,15 (the group's even bytes are the first eight
    k, its odd bytes the last eight)."""
    w_kn = np.ascontiguousarray(w_kn)
    k, n = w_kn.shape
    check_shape(k, n)
    w_nk = w_kn.T.reshape(n, k // 16, 16)
    order = np.array([0, 8, 1, 9, 2, 10, 3, 11, 4, 12, 5, 13, 6, 14, 7, 15])
    nn = np.arange(n)[:, None]
    jj = np.arange(k // 16)[None, :]
    off = (nn // 2) * 2 * k + ((16 * jj) // 64) * 128 + (nn % 2) * 64 + (16 * jj) % 64
    out = np.empty(k * n, dtype=w_kn.dtype)
    out[(off[:, :, None] + np.arange(16)[None, None, :]).reshape(-1)] = \
        w_nk[:, :, order].reshape(-1)
    return out.reshape(k, n)
