// dt_mx_fp8_bf16: block-scaled e4m3 x e4m3 -> bf16 GEMM (C ABI), and the GEMMs' split-K workspace.
// The kernel is in mx_gemm_kernels.hpp; the e2m1 entry points are compiled from mx_fp4_bf16.hip.
#include "mx_gemm_kernels.hpp"

extern "C" int dt_mx_fp8_bf16(const void* a, const void* b, const uint8_t* sfa, const uint8_t* sfb, int64_t M,
                              int64_t N, int64_t K, int64_t lda, int64_t ldb, void* out, int64_t ldo,
                              dt_stream_t stream) {
  return dt::mx_gemm<false>(a, b, sfa, sfb, M, N, K, lda, ldb, out, ldo, nullptr, 0, stream);
}

extern "C" size_t dt_mx_gemm_workspace_bytes(void) { return dt::split_workspace_bytes(); }

namespace dt {
__global__ void zero_tickets_kernel(uint32_t* p) { p[threadIdx.x] = 0u; }
}  // namespace dt

extern "C" int dt_mx_gemm_workspace_init(void* workspace, size_t workspace_bytes, dt_stream_t stream) {
  if (!workspace) return DT_ERR_NULL_POINTER;
  if (workspace_bytes < dt::kSplitTicketBytes) return DT_ERR_WORKSPACE;
  if (!dt::aligned(workspace, 256)) return DT_ERR_MISALIGNED;
  // a fill kernel rather than hipMemsetAsync, so the call is safe under graph capture
  dt::zero_tickets_kernel<<<1, dt::kSplitTicketBytes / 4, 0, dt::as_hip(stream)>>>(static_cast<uint32_t*>(workspace));
  return dt::launch_status();
}

extern "C" int dt_mx_fp8_bf16_ws(const void* a, const void* b, const uint8_t* sfa, const uint8_t* sfb, int64_t M,
                                 int64_t N, int64_t K, int64_t lda, int64_t ldb, void* out, int64_t ldo,
                                 void* workspace, size_t workspace_bytes, dt_stream_t stream) {
  return dt::mx_gemm<false>(a, b, sfa, sfb, M, N, K, lda, ldb, out, ldo, workspace, workspace_bytes, stream);
}
