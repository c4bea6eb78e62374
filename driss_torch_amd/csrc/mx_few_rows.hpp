// The block-scaled GEMM for problems of at most 64 rows (mx_few_rows.hip): what mx_fp8_bf16.hip needs of it.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dt {

// Can the kernel for few rows take the problem at all (M <= 64 and a K its 32-bit offsets span)?
bool few_rows_fits(int64_t M, int64_t K);

// Does the kernel for few rows beat the tiles for this problem?  (fp4: e2m1 operands; K counts elements.)
bool few_rows_pays(bool fp4, int64_t M, int64_t N, int64_t K, bool have_workspace);

// M <= 64; operands as for dt_mx_fp8_bf16 / dt_mx_fp4_bf16, already checked.  Returns a dt_status.
int launch_few_rows(bool fp4, const uint8_t* a, const uint8_t* b, const uint8_t* sfa, const uint8_t* sfb, int64_t M,
                    int64_t N, int64_t K, int64_t lda, int64_t ldb, void* out, int64_t ldo, hipStream_t stream);

}  // namespace dt
