// Internal interface of the fp32 MFMA GEMM (gemm_f32.hip), shared with the Winograd path.
#pragma once
#include "tsx_common.hpp"

namespace tsx {

// Strided-batch C[b] = A[b] * B[b]: A [m][k] row-major, B element (k, n) at b[k*ld_k + n*ld_n],
// C [m][n] row-major; batch b adds a_batch / b_batch / c_batch elements to the bases.
int gemm_f32_batched(const float *a, int64_t a_batch, const float *b, int64_t ld_k, int64_t ld_n, int64_t b_batch,
                     float *c, int64_t c_batch, int m, int n, int k, int batches, hipStream_t stream);

}  // namespace tsx
