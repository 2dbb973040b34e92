// extern "C" entry points of the GPTQ quantized linear: argument checks and
// the choice between the VALU GEMV, the MFMA GEMM and the generic fallback.
#include "gptq_common.h"

#include <pthread.h>

namespace mh {
bool gemv_supported(int M, int N, int K, int group_size, int bits);
size_t gemv_workspace_bytes(int M, int N, int K, int group_size, int bits);
int gptq_gemv_launch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                     const void* scales, void* out, int M, int N, int K, int group_size, int bits,
                     void* workspace, size_t workspace_bytes);
bool gemm_supported(int M, int N, int K, int group_size, int bits);
size_t gemm_workspace_bytes(int M, int N, int K, int group_size, int bits);
bool gemm_silu_pairs_supported(int M, int N, int K, int group_size, int bits);
bool gemm_tall_silu_pairs_supported(int M, int N, int K, int group_size, int bits);
int gptq_gemm_launch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                     const void* scales, void* out, int M, int N, int K, int group_size, int bits,
                     void* workspace, size_t workspace_bytes, int epilogue, const SmallFuse& fuse);
int gptq_generic_launch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                        const void* scales, const int32_t* g_idx, void* out, int M, int N, int K,
                        int group_size, int bits);
int gemv_gemm_crossover();
bool gemm_bias_supported(int M, int N, int K, int group_size, int bits);
int silu_pairs_launch(hipStream_t stream, const void* gate_up, void* out, int rows, int ffn);  // decode.hip
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

// ---- the product for callers that cannot allocate -----------------------------------------
// mh_gptq_matmul_static keeps the split-K workspace (arrival counters + fp32 partial sums) in
// device memory that belongs to the library: a file-scope array, one copy per GPU, held until
// the process ends.  In host code the array's name is only a handle for the runtime; the
// address kernels and fills may use comes from hipGetSymbolAddress, once per device.
namespace mh {
constexpr size_t kStaticScratchBytes = (size_t)MH_GPTQ_STATIC_SCRATCH_BYTES;
constexpr int kStaticMaxDevices = 64;
}  // namespace mh
static __device__ __align__(256) unsigned char scratch[mh::kStaticScratchBytes];

namespace mh {
static void* g_static_scratch[kStaticMaxDevices];   // device address of `scratch` per GPU, 0 = not looked up yet
static pthread_mutex_t g_static_lock = PTHREAD_MUTEX_INITIALIZER;

__global__ void static_scratch_clear_kernel(uint4* p, int n16) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n16) p[i] = make_uint4(0u, 0u, 0u, 0u);
}

// The current device's copy of `scratch` (looked up on first use on that device).  The lookup loads
// the code object's symbol table: not something to do while `stream` is being captured.
static int static_scratch_pointer(hipStream_t stream, void** out) {
    int dev = 0;
    MH_CHECK_HIP(hipGetDevice(&dev));
    MH_REQUIRE(dev >= 0 && dev < kStaticMaxDevices, "mh_gptq_matmul_static: device index %d out of range", dev);
    pthread_mutex_lock(&g_static_lock);
    void* ptr = g_static_scratch[dev];
    hipError_t err = hipSuccess;
    if (ptr == nullptr) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (stream != nullptr && hipStreamIsCapturing(stream, &capturing) == hipSuccess &&
            capturing != hipStreamCaptureStatusNone) {
            pthread_mutex_unlock(&g_static_lock);
            return fail(MH_ERR_INVALID, "mh_gptq_matmul_static: the first call on a device must be made outside a "
                                        "stream capture (it looks up the built-in buffer's address)");
        }
        err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err == hipSuccess) g_static_scratch[dev] = ptr;
    }
    pthread_mutex_unlock(&g_static_lock);
    if (err != hipSuccess || ptr == nullptr)
        return fail(MH_ERR_HIP, "mh_gptq_matmul_static: hipGetSymbolAddress(scratch): %s", hipGetErrorString(err));
    *out = ptr;
    return MH_OK;
}
}  // namespace mh

using namespace mh;

extern "C" {

size_t mh_gptq_static_scratch_bytes(void) { return kStaticScratchBytes; }

int mh_gptq_matmul_static(mh_stream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                          const void* scales, const int32_t* g_idx, void* out, int M, int N, int K,
                          int group_size, int bits) {
    int rc = check_gptq_args("mh_gptq_matmul_static", x, qweight, qzeros, scales, out, M, N, K, group_size, bits);
    if (rc) return rc;
    if (M == 0) return MH_OK;
    const size_t need = g_idx == nullptr ? mh_gptq_workspace_bytes(M, N, K, group_size, bits) : 0;
    if (need > kStaticScratchBytes)
        return fail(MH_ERR_WORKSPACE,
                    "mh_gptq_matmul_static: M=%d N=%d K=%d needs %zu bytes of split-K scratch, the built-in buffer "
                    "holds %zu; use mh_gptq_matmul with a caller-owned workspace",
                    M, N, K, need, kStaticScratchBytes);
    void* ws = nullptr;
    if (need != 0) {
        rc = static_scratch_pointer(as_stream(stream), &ws);
        if (rc) return rc;
        // the arrival counters must start at zero; the buffer keeps whatever the previous call (or a call
        // that was interrupted) left, so clear them with a kernel (no memset node, safe under graph capture)
        const int n16 = (int)(kTileCounterBytes / 16);
        static_scratch_clear_kernel<<<(n16 + 255) / 256, 256, 0, as_stream(stream)>>>(static_cast<uint4*>(ws), n16);
        MH_CHECK_LAUNCH();
    }
    return mh_gptq_matmul(stream, x, qweight, qzeros, scales, g_idx, out, M, N, K, group_size, bits, ws,
                          ws ? kStaticScratchBytes : 0);
}

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
               "mh_gptq_gemm: needs N %% 8 == 0, K %% 32 == 0, group_size %% 32 == 0 and packed weights below 2 GiB "
               "(M=%d N=%d K=%d g=%d)",
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

// Where the plain product sits in the workspace of the two-pass SiLU-pairs path: behind what the
// product itself needs, and never on the arrival counters at the head of a workspace (they must
// stay zero for every later call that shares the buffer, also when this product needs none).
static size_t silu_pairs_product_offset(size_t product_bytes) {
    const size_t floor = product_bytes > kTileCounterBytes ? product_bytes : kTileCounterBytes;
    return (floor + 255) / 256 * 256;
}

size_t mh_gptq_silu_pairs_workspace_bytes(int M, int N, int K, int group_size, int bits) {
    const size_t product = mh_gptq_workspace_bytes(M, N, K, group_size, bits);
    if (gemm_silu_pairs_supported(M, N, K, group_size, bits) || gemm_tall_silu_pairs_supported(M, N, K, group_size, bits))
        return product;
    return silu_pairs_product_offset(product) + (size_t)M * N * sizeof(half_t);
}

int mh_gptq_linear(mh_stream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                   const void* scales, const int32_t* g_idx, const void* bias, void* out, int M, int N, int K,
                   int group_size, int bits, void* workspace, size_t workspace_bytes) {
    if (bias == nullptr)
        return mh_gptq_matmul(stream, x, qweight, qzeros, scales, g_idx, out, M, N, K, group_size, bits, workspace,
                              workspace_bytes);
    int rc = check_gptq_args("mh_gptq_linear", x, qweight, qzeros, scales, out, M, N, K, group_size, bits);
    if (rc) return rc;
    if (M == 0) return MH_OK;
    const bool gemv = M <= gemv_gemm_crossover() && gemv_supported(M, N, K, group_size, bits);
    if (g_idx == nullptr && !gemv && gemm_bias_supported(M, N, K, group_size, bits)) {
        SmallFuse fuse;  // the bias rides on the product's own stores: one launch (two with a split-K second stage)
        fuse.bias = static_cast<const half_t*>(bias);
        return gptq_gemm_launch(as_stream(stream), x, qweight, qzeros, scales, out, M, N, K, group_size, bits,
                                workspace, workspace_bytes, kEpilogueNone, fuse);
    }
    rc = mh_gptq_matmul(stream, x, qweight, qzeros, scales, g_idx, out, M, N, K, group_size, bits, workspace,
                        workspace_bytes);
    if (rc) return rc;
    return mh_add_bias(stream, out, bias, (size_t)M, (size_t)N, MH_F16);
}

int mh_gptq_matmul_silu_pairs(mh_stream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                              const void* scales, void* out, int M, int N, int K, int group_size, int bits,
                              void* workspace, size_t workspace_bytes) {
    int rc = check_gptq_args("mh_gptq_matmul_silu_pairs", x, qweight, qzeros, scales, out, M, N, K, group_size, bits);
    if (rc) return rc;
    if (M == 0) return MH_OK;
    MH_REQUIRE(N % 256 == 0, "mh_gptq_matmul_silu_pairs: N=%d must be a multiple of 256 (128 gate + 128 up columns per block)", N);
    // up to 64 rows in the small-M kernel's reduction, above in the store of the 128-row blocks when K is unsplit
    if (gemm_silu_pairs_supported(M, N, K, group_size, bits) || gemm_tall_silu_pairs_supported(M, N, K, group_size, bits))
        return gptq_gemm_launch(as_stream(stream), x, qweight, qzeros, scales, out, M, N, K, group_size, bits,
                                workspace, workspace_bytes, kEpilogueSiluPairs, SmallFuse{});
    // more rows (or a group size) than either serves: the product into the workspace,
    // then one pass that applies silu(gate) * up to the fp16-rounded sums
    const size_t product = silu_pairs_product_offset(mh_gptq_workspace_bytes(M, N, K, group_size, bits));
    const size_t need = product + (size_t)M * N * sizeof(half_t);
    if (workspace == nullptr || workspace_bytes < need)
        return fail(MH_ERR_WORKSPACE, "mh_gptq_matmul_silu_pairs: workspace of %zu bytes required, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    half_t* gu = reinterpret_cast<half_t*>(static_cast<char*>(workspace) + product);
    rc = mh_gptq_matmul(stream, x, qweight, qzeros, scales, nullptr, gu, M, N, K, group_size, bits, workspace, product);
    if (rc) return rc;
    return silu_pairs_launch(as_stream(stream), gu, out, M, N / 2);
}

}  // extern "C"
