/*
 * dq8_test_hooks.h -- entry points of libdisc_q8_ral.so that exist for the tests and for
 * tuning only: they force one kernel variant where the library would choose, and expose the
 * MFMA register layouts to a brute-force check.  Not part of the product ABI (include/).
 */
#ifndef DQ8_TEST_HOOKS_H_
#define DQ8_TEST_HOOKS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dq8_qgemm (include/disc_q8.h), forcing one kernel variant:
 *  -1 heuristic, 0 generic scalar kernel, 1.. MFMA tile configurations
 *  (dq8_qgemm_num_variants() of them, names from dq8_qgemm_variant_name()).  A problem
 *  an MFMA variant cannot take (unaligned rows; K % 16 != 0 without scratch) runs on the
 *  generic kernel whatever the variant; non-zero zx / zw with a forced MFMA variant is an error
 *  (they need the heuristic or the generic variant). */
int dq8_qgemm_variant(int variant, const int8_t* A, int64_t lda,
                      const int8_t* W, int64_t ldw, void* out, int64_t ldo,
                      int64_t M, int64_t N, int64_t K, int tp_a, int tp_b,
                      int epilogue, const void* bias, int bias_kind,
                      const float* sx, int64_t n_sx, const float* sw,
                      int64_t n_sw, const float* so, int64_t n_so, int32_t zx,
                      int32_t zw, int32_t zo, void* workspace,
                      size_t workspace_bytes, void* stream);
int dq8_qgemm_num_variants(void);
const char* dq8_qgemm_variant_name(int variant);


/* dq8_qconv2d_ws (include/disc_q8.h), forcing one kernel variant (numbering as above). */
int dq8_qconv2d_variant(int variant, const int8_t* in,
                        const int64_t in_sizes[4], const int8_t* w,
                        const int64_t w_sizes[4], const int32_t padding[4],
                        const int32_t metadata[17], void* out,
                        const int64_t out_sizes[4], int epilogue,
                        const void* bias, int bias_kind, const float* sx,
                        const float* sw, int64_t n_sw, const float* so,
                        int32_t zo, void* workspace, size_t workspace_bytes,
                        void* stream);

/* Runs one v_mfma_i32_32x32x32_i8 and one v_mfma_i32_16x16x64_i8 on device
 * buffers: a[32*32] (row i, k contiguous), b[32*32] (column j, k contiguous) ->
 * d32[32*32] row-major; a16[16*64], b16[16*64] -> d16[16*16].  Lets a test pin
 * the operand and result register layouts against brute force. */
int dq8_mfma_probe(const int8_t* a, const int8_t* b, int32_t* d32,
                   const int8_t* a16, const int8_t* b16, int32_t* d16,
                   void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DQ8_TEST_HOOKS_H_ */
