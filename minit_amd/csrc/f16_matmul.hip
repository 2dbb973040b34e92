// Dense fp16 product with the reference's operand orientation:
//   out[m, n] = fp16( sum_k fp32(a[m, k]) * fp32(b[n, k]) ),  b stored [N, K]
// (dispatch_matmul + minit_gemm, minit/cuda/dispatch.py:59-78,
// minit/cuda/kernel/cublas.py:68-111).  Used for the unquantized lm_head at
// decode and as the dense leg of the act-order path.
//
// Both operands are K-contiguous, which is the MFMA operand layout as is: lane l
// of a 16x16x32 fp16 MFMA holds eight consecutive k of row l % 16, k-chunk l / 16,
// i.e. one 16-byte load straight from global memory for either operand.  A wave
// owns 16 rows of b (16 output columns) for all of K; b is streamed once, a is
// small and served by the caches.
#include "common.h"

namespace mh {

constexpr int kDenseDepth = 8;

// Both operands travel through a ring of kDenseDepth steps of registers that is
// refilled one slot per step at a fixed place of a branch-free loop body, so the
// compiler can wait with an exact vmcnt and the stream of b never drains.  (With
// the a fragment fetched at its point of use, every step waited for the load it
// had just issued.)  Steps past the end of K re-read the last step and multiply
// it by a zeroed a fragment.
template <int MT, int NT>
__global__ __launch_bounds__(256) void f16_matmul_nk_kernel(const half_t* __restrict__ a,
                                                            const half_t* __restrict__ b,
                                                            half_t* __restrict__ out, int M, int N, int K) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i16 = lane & 15, kq = lane >> 4;
    // a wave owns NT groups of 16 output columns: above 16 rows two groups share every
    // a fragment, which halves the a traffic per byte of b (a comes from the caches,
    // but through the same vector memory path as b)
    const int n0 = (blockIdx.x * 4 + wave) * (16 * NT);
    const int m0 = blockIdx.y * (16 * MT);
    if (n0 >= N) return;
    const half_t* brow[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) brow[nt] = b + (size_t)min(n0 + nt * 16 + i16, N - 1) * K + kq * 8;
    const half_t* arow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) arow[mt] = a + (size_t)min(m0 + mt * 16 + i16, M - 1) * K + kq * 8;

    float4_t acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int steps = K / 32;
    const int last = steps - 1;
    constexpr int D = kDenseDepth;
    uint4_t bq[D][NT], aq[D][MT];
    auto load = [&](int slot, int s) {
        const size_t off = (size_t)min(s, last) * 32;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            bq[slot][nt] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(brow[nt] + off));
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) aq[slot][mt] = *reinterpret_cast<const uint4_t*>(arow[mt] + off);
    };
#pragma unroll
    for (int d = 0; d < D; ++d) load(d, d);
    for (int s0 = 0; s0 < steps; s0 += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const bool live = s0 + d <= last;
            half8_t bf[NT], af[MT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) bf[nt] = __builtin_bit_cast(half8_t, bq[d][nt]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                af[mt] = __builtin_bit_cast(half8_t, live ? aq[d][mt] : uint4_t{0u, 0u, 0u, 0u});
            load(d, s0 + d + D);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)  // rows of the result are m (operand A), columns are n (operand B)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[mt], bf[nt], acc[mt][nt], 0, 0, 0);
        }
    }
    // acc[mt][nt][r] is row m0 + mt*16 + kq*4 + r, column n0 + nt*16 + i16
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int n = n0 + nt * 16 + i16;
        if (n >= N) continue;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + mt * 16 + kq * 4 + r;
                if (m < M) out[(size_t)m * N + n] = (half_t)acc[mt][nt][r];
            }
    }
}

// Any K (no divisibility or alignment assumptions): one thread per output.
__global__ void f16_matmul_nk_generic_kernel(const half_t* __restrict__ a, const half_t* __restrict__ b,
                                             half_t* __restrict__ out, int M, int N, int K) {
    const size_t total = (size_t)M * N;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
        const int m = (int)(idx / N), n = (int)(idx % N);
        float acc = 0.f;
        for (int k = 0; k < K; ++k) acc = __builtin_fmaf((float)a[(size_t)m * K + k], (float)b[(size_t)n * K + k], acc);
        out[idx] = (half_t)acc;
    }
}

}  // namespace mh

using namespace mh;

extern "C" int mh_f16_matmul_nk(mh_stream_t stream, const void* a, const void* b, void* out, int M, int N,
                                int K) {
    MH_REQUIRE(M >= 0 && N >= 0 && K >= 0, "mh_f16_matmul_nk: bad shape M=%d N=%d K=%d", M, N, K);
    if (M == 0 || N == 0) return MH_OK;
    MH_REQUIRE(a && b && out, "mh_f16_matmul_nk: null pointer");
    hipStream_t st = as_stream(stream);
    const bool fast = K > 0 && K % 32 == 0 && ((uintptr_t)a | (uintptr_t)b) % 16 == 0;
    if (!fast) {
        size_t blocks = ((size_t)M * N + 255) / 256;
        const size_t cap = (size_t)compute_units() * 16;
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL(f16_matmul_nk_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, st,
                           (const half_t*)a, (const half_t*)b, (half_t*)out, M, N, K);
        MH_CHECK_LAUNCH();
        return MH_OK;
    }
    const int mt = M <= 16 ? 1 : M <= 32 ? 2 : 4;
    const int nt = mt == 1 ? 1 : 2;  // columns per wave: 16 or 32
    dim3 grid((N + 64 * nt - 1) / (64 * nt), (M + 16 * mt - 1) / (16 * mt));
#define MH_DENSE(MT, NT)                                                                                            \
    hipLaunchKernelGGL((f16_matmul_nk_kernel<MT, NT>), grid, dim3(256), 0, st, (const half_t*)a, (const half_t*)b, \
                       (half_t*)out, M, N, K)
    switch (mt) {
        case 1: MH_DENSE(1, 1); break;
        case 2: MH_DENSE(2, 2); break;
        default: MH_DENSE(4, 2); break;
    }
#undef MH_DENSE
    MH_CHECK_LAUNCH();
    return MH_OK;
}
