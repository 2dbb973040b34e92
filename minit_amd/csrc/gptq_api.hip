// extern "C" entry points of the GPTQ quantized linear: argument checks and
// the choice between the VALU GEMV, the MFMA GEMM and the generic fallback.
#include "gptq_common.h"

namespace mh {
bool gemv_supported(int M, int N, int K, int group_size, int bits);
size_t gemv_workspace_bytes(int M, int N, int K, int group_size, int bits);
int gptq_gemv_launch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                     const void* scales, void* out, int M, int N, int K, int group_size, int bits,
                     void* workspace, size_t workspace_bytes);
bool gemm_supported(int M, int N, int K, int group_size, int bits);
size_t gemm_workspace_bytes(int M, int N, int K, int group_size, int bits);
bool gemm_silu_pairs_supported(int M, int N, int K, int group_size, int bits);
int gptq_gemm_launch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                     const void* scales, void* out, int M, int N, int K, int group_size, int bits,
                     void* workspace, size_t workspace_bytes, int epilogue, const SmallFuse& fuse);
int gptq_generic_launch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                        const void* scales, const int32_t* g_idx, void* out, int M, int N, int K,
                        int group_size, int bits);
int gemv_gemm_crossover();
}  // namespace mh

namespace mh {
// Trusted-argument path for callers inside the library (the decode loop).
int gptq_matmul_dispatch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                         const void* scales, void* out, int M, int N, int K, int group_size, int bits,
                         void* workspace, size_t workspace_bytes) {
    if (M <= gemv_gemm_crossover() && gemv_supported(M, N, K, group_size, bits))
        return gptq_gemv_launch(stream, x, qweight, qzeros, scales, out, M, N, K, group_size, bits, workspace,
                                workspace_bytes);
    if (gemm_supported(M, N, K, group_size, bits))
        return gptq_gemm_launch(stream, x, qweight, qzeros, scales, out, M, N, K, group_size, bits, workspace,
                                workspace_bytes, kEpilogueNone, SmallFuse{});
    return gptq_generic_launch(stream, x, qweight, qzeros, scales, nullptr, out, M, N, K, group_size, bits);
}

// out [M, N / 2] = silu(gate) * up of the product, for weights whose column tiles
// interleave gate and up (kEpilogueSiluPairs); the caller has checked
// gemm_silu_pairs_supported().
int gptq_matmul_silu_pairs(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                           const void* scales, void* out, int M, int N, int K, int group_size, int bits,
                           void* workspace, size_t workspace_bytes) {
    return gptq_gemm_launch(stream, x, qweight, qzeros, scales, out, M, N, K, group_size, bits, workspace,
                            workspace_bytes, kEpilogueSiluPairs, SmallFuse{});
}

// The product with the fusions of SmallFuse / an epilogue chosen by the caller
// (the decode loop); the caller has checked the *_supported() predicate.
int gptq_matmul_fused(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                      const void* scales, void* out, int M, int N, int K, int group_size, int bits,
                      void* workspace, size_t workspace_bytes, int epilogue, const SmallFuse& fuse) {
    return gptq_gemm_launch(stream, x, qweight, qzeros, scales, out, M, N, K, group_size, bits, workspace,
                            workspace_bytes, epilogue, fuse);
}
}  // namespace mh

using namespace mh;

extern "C" {

size_t mh_gptq_workspace_bytes(int M, int N, int K, int group_size, int bits) {
    if (M <= 0 || N <= 0 || K <= 0 || group_size <= 0 || (bits != 4 && bits != 8)) return 0;
    if (K % group_size != 0 || group_size % (32 / bits) != 0 || N % 8 != 0) return 0;
    size_t a = 0, b = 0;
    if (gemv_supported(M, N, K, group_size, bits)) a = gemv_workspace_bytes(M, N, K, group_size, bits);
    if (gemm_supported(M, N, K, group_size, bits)) b = gemm_workspace_bytes(M, N, K, group_size, bits);
    return a > b ? a : b;
}

int mh_gptq_gemv(mh_stream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                 const void* scales, const int32_t* g_idx, void* out, int M, int N, int K,
                 int group_size, int bits, void* workspace, size_t workspace_bytes) {
    int rc = check_gptq_args("mh_gptq_gemv", x, qweight, qzeros, scales, out, M, N, K, group_size, bits);
    if (rc) return rc;
    if (M == 0) return MH_OK;
    MH_REQUIRE(g_idx == nullptr, "mh_gptq_gemv: act-order g_idx is served by mh_gptq_matmul");
    MH_REQUIRE(gemv_supported(M, N, K, group_size, bits),
               "mh_gptq_gemv: needs 1 <= M <= %d, N %% 8 == 0, group_size %% %d == 0 (M=%d N=%d K=%d g=%d)",
               MH_GPTQ_GEMV_MAX_M, 32 / bits, M, N, K, group_size);
    return gptq_gemv_launch(as_stream(stream), x, qweight, qzeros, scales, out, M, N, K, group_size, bits,
                            workspace, workspace_bytes);
}

int mh_gptq_gemm(mh_stream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                 const void* scales, const int32_t* g_idx, void* out, int M, int N, int K,
                 int group_size, int bits, void* workspace, size_t workspace_bytes) {
    int rc = check_gptq_args("mh_gptq_gemm", x, qweight, qzeros, scales, out, M, N, K, group_size, bits);
    if (rc) return rc;
    if (M == 0) return MH_OK;
    MH_REQUIRE(g_idx == nullptr, "mh_gptq_gemm: act-order g_idx is served by mh_gptq_matmul");
    MH_REQUIRE(gemm_supported(M, N, K, group_size, bits),
               "mh_gptq_gemm: needs N %% 8 == 0, K %% 32 == 0, group_size %% 32 == 0 (M=%d N=%d K=%d g=%d)",
               M, N, K, group_size);
    return gptq_gemm_launch(as_stream(stream), x, qweight, qzeros, scales, out, M, N, K, group_size, bits,
                            workspace, workspace_bytes, kEpilogueNone, SmallFuse{});
}

int mh_gptq_matmul(mh_stream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                   const void* scales, const int32_t* g_idx, void* out, int M, int N, int K,
                   int group_size, int bits, void* workspace, size_t workspace_bytes) {
    int rc = check_gptq_args("mh_gptq_matmul", x, qweight, qzeros, scales, out, M, N, K, group_size, bits);
    if (rc) return rc;
    if (M == 0) return MH_OK;
    if (g_idx == nullptr) {
        if (M <= gemv_gemm_crossover() && gemv_supported(M, N, K, group_size, bits))
            return gptq_gemv_launch(as_stream(stream), x, qweight, qzeros, scales, out, M, N, K, group_size,
                                    bits, workspace, workspace_bytes);
        if (gemm_supported(M, N, K, group_size, bits))
            return gptq_gemm_launch(as_stream(stream), x, qweight, qzeros, scales, out, M, N, K, group_size,
                                    bits, workspace, workspace_bytes, kEpilogueNone, SmallFuse{});
    }
    return gptq_generic_launch(as_stream(stream), x, qweight, qzeros, scales, g_idx, out, M, N, K,
                               group_size, bits);
}

int mh_gptq_matmul_silu_pairs(mh_stream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                              const void* scales, void* out, int M, int N, int K, int group_size, int bits,
                              void* workspace, size_t workspace_bytes) {
    int rc = check_gptq_args("mh_gptq_matmul_silu_pairs", x, qweight, qzeros, scales, out, M, N, K, group_size, bits);
    if (rc) return rc;
    if (M == 0) return MH_OK;
    return gptq_gemm_launch(as_stream(stream), x, qweight, qzeros, scales, out, M, N, K, group_size, bits,
                            workspace, workspace_bytes, kEpilogueSiluPairs, SmallFuse{});
}

}  // extern "C"
