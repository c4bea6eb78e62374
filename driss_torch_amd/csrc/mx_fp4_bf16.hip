// dt_mx_fp4_bf16: block-scaled e2m1 x e2m1 -> bf16 GEMM (C ABI): the FP4 instantiations of the kernel in
// mx_gemm_kernels.hpp, compiled on their own so that the two operand types build side by side.
#include "mx_gemm_kernels.hpp"

extern "C" int dt_mx_fp4_bf16(const void* a, const void* b, const uint8_t* sfa, const uint8_t* sfb, int64_t M,
                              int64_t N, int64_t K, int64_t lda, int64_t ldb, void* out, int64_t ldo,
                              dt_stream_t stream) {
  return dt::mx_gemm<true>(a, b, sfa, sfb, M, N, K, lda, ldb, out, ldo, nullptr, 0, stream);
}

extern "C" int dt_mx_fp4_bf16_ws(const void* a, const void* b, const uint8_t* sfa, const uint8_t* sfb, int64_t M,
                                 int64_t N, int64_t K, int64_t lda, int64_t ldb, void* out, int64_t ldo,
                                 void* workspace, size_t workspace_bytes, dt_stream_t stream) {
  return dt::mx_gemm<true>(a, b, sfa, sfb, M, N, K, lda, ldb, out, ldo, workspace, workspace_bytes, stream);
}
