// W8A8 int8 GEMM on CDNA4 int8 MFMA (v_mfma_i32_32x32x32_i8) with exact int32
// accumulation and a per-token x per-channel scale epilogue.
//
// The reference has no int8 x int8 product; the operand orientation is the one
// of its dense MatrixMultiply, C[m, n] = sum_k A[m, k] * B[n, k]
// (minit/operator/linalg.py:29-35, minit/cuda/kernel/cublas.py:83), so both
// operands are K-contiguous -- exactly what the MFMA operand layout wants
// (16 consecutive k per lane).
//
// Tiling: block tile 128 x 256 x 64, four waves in a 2 x 2 arrangement, each
// computing 64 x 128 as 2 x 4 MFMA tiles of 32 x 32.  Operand tiles are staged
// through LDS with a 16-byte-chunk XOR swizzle (rows are 64 bytes, so unswizzled
// ds_read_b128 of 8 consecutive rows would hit the same banks), double
// buffered, with the next stage held in registers while the current one is
// consumed: one barrier per 64-k step.  blockIdx -> tile mapping is XCD-aware:
// consecutive block ids land on different XCDs, so each XCD is given a compact
// rectangle of tiles and its L2 sees each operand row few times.
#include "common.h"

namespace mh {

constexpr int kI8BM = 128, kI8BN = 256, kI8BK = 64;

__device__ __forceinline__ int swz(int row, int chunk) { return row * 64 + ((chunk ^ ((row >> 1) & 3)) << 4); }

__global__ __launch_bounds__(256) void i8_gemm_kernel(
    const int8_t* __restrict__ A, const int8_t* __restrict__ W, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, half_t* __restrict__ out, int32_t* __restrict__ acc_out,
    int M, int N, int K, int tiles_m, int tiles_n, int group_m, int xcd_chunk) {
    __shared__ __attribute__((aligned(16))) int8_t As[2][kI8BM * kI8BK];
    __shared__ __attribute__((aligned(16))) int8_t Bs[2][kI8BN * kI8BK];

    // XCD-aware tile order: block b runs on XCD b % 8; give every XCD a run of
    // xcd_chunk consecutive positions of a grouped (group_m rows at a time) order.
    int o = blockIdx.x;
    if (xcd_chunk > 0) o = (o % 8) * xcd_chunk + o / 8;
    const int per_group = group_m * tiles_n;
    const int grp = o / per_group;
    const int first_m = grp * group_m;
    const int rows_here = min(group_m, tiles_m - first_m);
    const int in_grp = o % per_group;
    const int tm = first_m + in_grp % rows_here;
    const int tn = in_grp / rows_here;
    const int m0 = tm * kI8BM, n0 = tn * kI8BN;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wy = wave >> 1, wx = wave & 1;
    const int l32 = lane & 31, lh = lane >> 5;

    int16_t_v acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    // staging: A has 512 chunks (2 per thread), B has 1024 (4 per thread)
    int4_t ra[2], rb[4];
    const int crow = tid >> 2, cchunk = tid & 3;  // +64 rows per extra chunk
    auto load_stage = [&](int k0) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int m = min(m0 + crow + 64 * j, M - 1);
            ra[j] = *reinterpret_cast<const int4_t*>(A + (size_t)m * K + k0 + cchunk * 16);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = min(n0 + crow + 64 * j, N - 1);
            rb[j] = *reinterpret_cast<const int4_t*>(W + (size_t)n * K + k0 + cchunk * 16);
        }
    };
    auto store_stage = [&](int buf) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
            *reinterpret_cast<int4_t*>(&As[buf][swz(crow + 64 * j, cchunk)]) = ra[j];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            *reinterpret_cast<int4_t*>(&Bs[buf][swz(crow + 64 * j, cchunk)]) = rb[j];
    };

    const int KT = K / kI8BK;
    load_stage(0);
    store_stage(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < KT) load_stage((kt + 1) * kI8BK);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int chunk = ks * 2 + lh;
            int4_t a[2], b[4];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                a[i] = *reinterpret_cast<const int4_t*>(&As[buf][swz(wy * 64 + i * 32 + l32, chunk)]);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                b[j] = *reinterpret_cast<const int4_t*>(&Bs[buf][swz(wx * 128 + j * 32 + l32, chunk)]);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < KT) store_stage(buf ^ 1);
        __syncthreads();
    }

    // epilogue: acc[i][j][r] is row (r/4)*8 + lh*4 + r%4, column l32 of its 32x32 tile
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + wx * 128 + j * 32 + l32;
            if (n >= N) continue;
            const float ws = w_scale ? w_scale[n] : 1.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wy * 64 + i * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                if (m >= M) continue;
                const int v = acc[i][j][r];
                if (acc_out) acc_out[(size_t)m * N + n] = v;
                if (out) {
                    const float s = (a_scale ? a_scale[m] : 1.f) * ws;
                    // The product is rounded to fp32 and only then to fp16; the
                    // empty asm keeps the compiler from fusing both into one
                    // mixed-precision instruction that rounds once.
                    float prod = (float)v * s;
                    asm volatile("" : "+v"(prod));
                    out[(size_t)m * N + n] = (half_t)prod;
                }
            }
        }
}

// out[c, r] = in[r, c] through a 64 x 64 LDS tile.
__global__ __launch_bounds__(256) void i8_transpose_kernel(const int8_t* __restrict__ in,
                                                           int8_t* __restrict__ out, int rows, int cols) {
    __shared__ int8_t tile[64][65];
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int i = ty; i < 64; i += 4) {
        const int r = r0 + i, c = c0 + tx;
        tile[i][tx] = (r < rows && c < cols) ? in[(size_t)r * cols + c] : (int8_t)0;
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
        const int c = c0 + i, r = r0 + tx;
        if (r < rows && c < cols) out[(size_t)c * rows + r] = tile[tx][i];
    }
}

}  // namespace mh

using namespace mh;

extern "C" {

int mh_i8_gemm(mh_stream_t stream, const int8_t* a, const int8_t* w, const float* a_scale,
               const float* w_scale, void* out_f16, int32_t* acc_i32, int M, int N, int K) {
    MH_REQUIRE(M >= 0 && N >= 0 && K > 0, "mh_i8_gemm: bad shape M=%d N=%d K=%d", M, N, K);
    if (M == 0 || N == 0) return MH_OK;
    MH_REQUIRE(K % kI8BK == 0, "mh_i8_gemm: K=%d must be a multiple of %d", K, kI8BK);
    MH_REQUIRE(a && w, "mh_i8_gemm: null operand");
    MH_REQUIRE(out_f16 || acc_i32, "mh_i8_gemm: no output requested");
    MH_REQUIRE(!out_f16 || (a_scale && w_scale), "mh_i8_gemm: scales required for the fp16 output");
    MH_REQUIRE(((uintptr_t)a | (uintptr_t)w) % 16 == 0, "mh_i8_gemm: operands must be 16-byte aligned");
    const int tiles_m = (M + kI8BM - 1) / kI8BM, tiles_n = (N + kI8BN - 1) / kI8BN;
    const int tiles = tiles_m * tiles_n;
    const int group_m = tiles_m < 8 ? tiles_m : 8;
    const int xcd_chunk = (tiles % 8 == 0) ? tiles / 8 : 0;
    hipLaunchKernelGGL(i8_gemm_kernel, dim3(tiles), dim3(256), 0, as_stream(stream), a, w, a_scale, w_scale,
                       (half_t*)out_f16, acc_i32, M, N, K, tiles_m, tiles_n, group_m, xcd_chunk);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

int mh_i8_transpose(mh_stream_t stream, const int8_t* in, int8_t* out, int rows, int cols) {
    MH_REQUIRE(rows >= 0 && cols >= 0, "mh_i8_transpose: bad shape");
    if (rows == 0 || cols == 0) return MH_OK;
    MH_REQUIRE(in && out, "mh_i8_transpose: null pointer");
    hipLaunchKernelGGL(i8_transpose_kernel, dim3((cols + 63) / 64, (rows + 63) / 64), dim3(256), 0,
                       as_stream(stream), in, out, rows, cols);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

}  // extern "C"
