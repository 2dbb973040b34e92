// GPTQ sub-word unpack, full dequantisation, and the shape-generic / act-order
// quantized matmul fallback.  These are the straightforward kernels; the
// bandwidth-tuned paths live in gptq_gemv.hip and gptq_gemm.hip.
#include "gptq_common.h"

namespace mh {

#pragma clang fp contract(off)

// out[r * P + i, c] (axis 0) or out[r, c * P + i] (axis 1) = sub-word i of packed[r, c].
// One thread per packed word; for axis 1 a thread writes P adjacent bytes.
template <int BITS>
__global__ void unpack_kernel(const uint32_t* __restrict__ packed, uint8_t* __restrict__ out,
                              size_t rows, size_t cols, int axis) {
    constexpr int P = Packing<BITS>::kPerWord;
    constexpr uint32_t MASK = Packing<BITS>::kMask;
    const size_t total = rows * cols;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
        const size_t r = idx / cols, c = idx % cols;
        const uint32_t q = packed[idx];
        if (axis == 0) {
#pragma unroll
            for (int i = 0; i < P; ++i) out[(r * P + i) * cols + c] = (uint8_t)((q >> (i * BITS)) & MASK);
        } else {
            uint8_t* o = out + (r * cols + c) * P;
#pragma unroll
            for (int i = 0; i < P; ++i) o[i] = (uint8_t)((q >> (i * BITS)) & MASK);
        }
    }
}

__device__ __forceinline__ half_t dequant_one(uint32_t q, uint32_t z, half_t s) {
    // (data.cast(f16) - (zero.cast(f16) + 1)) * scale, each step in fp16
    const half_t qf = (half_t)(float)q;
    const half_t zf = (half_t)(float)z + (half_t)1.0f;
    return (qf - zf) * s;
}

// One thread per packed word (r, n): writes P rows of column n.
template <int BITS>
__global__ void dequant_kernel(const uint32_t* __restrict__ qweight, const uint32_t* __restrict__ qzeros,
                               const half_t* __restrict__ scales, const int32_t* __restrict__ g_idx,
                               half_t* __restrict__ out, int N, int K, int group_size) {
    constexpr int P = Packing<BITS>::kPerWord;
    constexpr uint32_t MASK = Packing<BITS>::kMask;
    const size_t total = (size_t)(K / P) * N;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
        const int r = (int)(idx / N), n = (int)(idx % N);
        const uint32_t q = qweight[idx];
#pragma unroll
        for (int i = 0; i < P; ++i) {
            const int k = r * P + i;
            const int g = g_idx ? min(max(g_idx[k], 0), K / group_size - 1) : k / group_size;  // a bad index reads a wrong group, not outside the tables
            const uint32_t z = (qzeros[(size_t)g * (N / P) + n / P] >> ((n % P) * BITS)) & MASK;
            const half_t s = scales[(size_t)g * N + n];
            out[(size_t)k * N + n] = dequant_one((q >> (i * BITS)) & MASK, z, s);
        }
    }
}

// Shape-generic quantized matmul: thread per output column, block row per m.
// Handles a non-trivial g_idx (act-order) by looking the group up per k.
template <int BITS>
__global__ __launch_bounds__(256) void gptq_matmul_generic_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ qweight,
    const uint32_t* __restrict__ qzeros, const half_t* __restrict__ scales,
    const int32_t* __restrict__ g_idx, half_t* __restrict__ out, int N, int K, int group_size) {
    constexpr int P = Packing<BITS>::kPerWord;
    constexpr uint32_t MASK = Packing<BITS>::kMask;
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    const int m = blockIdx.y;
    if (n >= N) return;
    const half_t* xr = x + (size_t)m * K;
    float acc = 0.f;
    for (int r = 0; r < K / P; ++r) {
        const uint32_t q = qweight[(size_t)r * N + n];
#pragma unroll
        for (int i = 0; i < P; ++i) {
            const int k = r * P + i;
            const int g = g_idx ? min(max(g_idx[k], 0), K / group_size - 1) : k / group_size;  // a bad index reads a wrong group, not outside the tables
            const uint32_t z = (qzeros[(size_t)g * (N / P) + n / P] >> ((n % P) * BITS)) & MASK;
            const half_t w = dequant_one((q >> (i * BITS)) & MASK, z, scales[(size_t)g * N + n]);
            acc = __builtin_fmaf((float)xr[k], (float)w, acc);
        }
    }
    out[(size_t)m * N + n] = (half_t)acc;
}

int check_gptq_args(const char* who, const void* x, const void* qweight, const void* qzeros,
                    const void* scales, const void* out, int M, int N, int K, int group_size, int bits) {
    if (bits != 4 && bits != 8) return fail(MH_ERR_INVALID, "%s: bits must be 4 or 8, got %d", who, bits);
    const int P = 32 / bits;
    if (M < 0 || N <= 0 || K <= 0) return fail(MH_ERR_INVALID, "%s: bad shape M=%d N=%d K=%d", who, M, N, K);
    if (group_size <= 0 || K % group_size != 0)
        return fail(MH_ERR_INVALID, "%s: K=%d is not a multiple of group_size=%d", who, K, group_size);
    if (K % P != 0) return fail(MH_ERR_INVALID, "%s: K=%d is not a multiple of the pack size %d", who, K, P);
    if (N % P != 0) return fail(MH_ERR_INVALID, "%s: N=%d is not a multiple of the pack size %d", who, N, P);
    if (M > 0 && (!x || !out)) return fail(MH_ERR_INVALID, "%s: null activation or output pointer", who);
    if (!qweight || !qzeros || !scales) return fail(MH_ERR_INVALID, "%s: null weight pointer", who);
    if (((uintptr_t)qweight | (uintptr_t)scales | (uintptr_t)qzeros) % 16 != 0 ||
        ((uintptr_t)x | (uintptr_t)out) % 16 != 0)
        return fail(MH_ERR_INVALID, "%s: pointers must be 16-byte aligned", who);
    return MH_OK;
}

int gptq_generic_launch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                        const void* scales, const int32_t* g_idx, void* out, int M, int N, int K,
                        int group_size, int bits) {
    dim3 grid((N + 255) / 256, M), block(256);
    if (bits == 4)
        hipLaunchKernelGGL(gptq_matmul_generic_kernel<4>, grid, block, 0, stream, (const half_t*)x,
                           (const uint32_t*)qweight, (const uint32_t*)qzeros, (const half_t*)scales, g_idx,
                           (half_t*)out, N, K, group_size);
    else
        hipLaunchKernelGGL(gptq_matmul_generic_kernel<8>, grid, block, 0, stream, (const half_t*)x,
                           (const uint32_t*)qweight, (const uint32_t*)qzeros, (const half_t*)scales, g_idx,
                           (half_t*)out, N, K, group_size);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

// Rows of a packed weight in another order: out row j = in row perm[j], sub-word by sub-word
// (the one-time repack of an act-order checkpoint, rows sorted by group, so that the kernels
// that read sequential groups serve it).  One thread per output word.
template <int BITS>
__global__ void permute_rows_kernel(const uint32_t* __restrict__ packed, const int32_t* __restrict__ perm,
                                    uint32_t* __restrict__ out, size_t packed_rows, size_t cols) {
    constexpr int P = Packing<BITS>::kPerWord;
    constexpr uint32_t MASK = Packing<BITS>::kMask;
    const size_t total = packed_rows * cols;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t row = i / cols, col = i % cols;
        uint32_t word = 0;
#pragma unroll
        for (int e = 0; e < P; ++e) {
            // an index outside [0, K) reads the nearest row instead of memory outside the matrix
            const size_t src = (size_t)min(max(perm[row * P + e], 0), (int)(packed_rows * P) - 1);
            word |= ((packed[src / P * cols + col] >> (src % P * BITS)) & MASK) << (e * BITS);
        }
        out[i] = word;
    }
}

}  // namespace mh

using namespace mh;

extern "C" {

int mh_gptq_permute_rows(mh_stream_t stream, const int32_t* qweight, const int32_t* perm, int32_t* out, int N,
                         int K, int bits) {
    MH_REQUIRE(bits == 4 || bits == 8, "mh_gptq_permute_rows: bits must be 4 or 8, got %d", bits);
    MH_REQUIRE(N > 0 && K > 0 && K % (32 / bits) == 0, "mh_gptq_permute_rows: bad shape N=%d K=%d", N, K);
    MH_REQUIRE(qweight && perm && out && qweight != out, "mh_gptq_permute_rows: null pointer, or in place");
    const size_t packed_rows = (size_t)K / (32 / bits), total = packed_rows * N;
    size_t blocks = (total + 255) / 256;
    const size_t cap = (size_t)compute_units() * 16;
    if (blocks > cap) blocks = cap;
    if (bits == 4)
        hipLaunchKernelGGL(permute_rows_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           (const uint32_t*)qweight, perm, (uint32_t*)out, packed_rows, (size_t)N);
    else
        hipLaunchKernelGGL(permute_rows_kernel<8>, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           (const uint32_t*)qweight, perm, (uint32_t*)out, packed_rows, (size_t)N);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

int mh_gptq_unpack(mh_stream_t stream, const int32_t* packed, uint8_t* out, size_t rows, size_t cols,
                   int axis, int bits) {
    MH_REQUIRE(bits == 4 || bits == 8, "mh_gptq_unpack: bits must be 4 or 8, got %d", bits);
    MH_REQUIRE(axis == 0 || axis == 1, "mh_gptq_unpack: axis must be 0 or 1, got %d", axis);
    if (rows == 0 || cols == 0) return MH_OK;
    MH_REQUIRE(packed && out, "mh_gptq_unpack: null pointer");
    const size_t total = rows * cols;
    size_t blocks = (total + 255) / 256;
    const size_t cap = (size_t)compute_units() * 16;
    if (blocks > cap) blocks = cap;
    if (bits == 4)
        hipLaunchKernelGGL(unpack_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           (const uint32_t*)packed, out, rows, cols, axis);
    else
        hipLaunchKernelGGL(unpack_kernel<8>, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           (const uint32_t*)packed, out, rows, cols, axis);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

int mh_gptq_dequant(mh_stream_t stream, const int32_t* qweight, const int32_t* qzeros, const void* scales,
                    const int32_t* g_idx, void* out, int N, int K, int group_size, int bits) {
    int rc = check_gptq_args("mh_gptq_dequant", out, qweight, qzeros, scales, out, 1, N, K, group_size, bits);
    if (rc) return rc;
    const int P = 32 / bits;
    const size_t total = (size_t)(K / P) * N;
    size_t blocks = (total + 255) / 256;
    const size_t cap = (size_t)compute_units() * 16;
    if (blocks > cap) blocks = cap;
    if (bits == 4)
        hipLaunchKernelGGL(dequant_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           (const uint32_t*)qweight, (const uint32_t*)qzeros, (const half_t*)scales, g_idx,
                           (half_t*)out, N, K, group_size);
    else
        hipLaunchKernelGGL(dequant_kernel<8>, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           (const uint32_t*)qweight, (const uint32_t*)qzeros, (const half_t*)scales, g_idx,
                           (half_t*)out, N, K, group_size);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

}  // extern "C"
