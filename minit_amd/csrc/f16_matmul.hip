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
//
// KS = 4: the four waves of a workgroup share one group of 16 NT columns and take a quarter of K each
// (a weight of few rows gives too few waves for the memory system otherwise); their sums meet in LDS.
template <int MT, int NT, int KS>
__global__ __launch_bounds__(256) void f16_matmul_nk_kernel(const half_t* __restrict__ a,
                                                            const half_t* __restrict__ b,
                                                            half_t* __restrict__ out, int M, int N, int K) {
    // blockIdx.z: the matrix of a batch (a [batch, M, K], b [batch, N, K], out [batch, M, N])
    a += (size_t)blockIdx.z * M * K;
    b += (size_t)blockIdx.z * N * K;
    out += (size_t)blockIdx.z * M * N;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i16 = lane & 15, kq = lane >> 4;
    // a wave owns NT groups of 16 output columns: above 16 rows two groups share every
    // a fragment, which halves the a traffic per byte of b (a comes from the caches,
    // but through the same vector memory path as b)
    const int n0 = (KS == 1 ? blockIdx.x * 4 + wave : blockIdx.x) * (16 * NT);
    const int m0 = blockIdx.y * (16 * MT);
    if (n0 >= N) return;  // the whole workgroup when its waves share the columns
    const int steps = K / (32 * KS);  // of this wave
    const int k_first = KS == 1 ? 0 : wave * steps * 32;
    const half_t* brow[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) brow[nt] = b + (size_t)min(n0 + nt * 16 + i16, N - 1) * K + kq * 8 + k_first;
    const half_t* arow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) arow[mt] = a + (size_t)min(m0 + mt * 16 + i16, M - 1) * K + kq * 8 + k_first;

    float4_t acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int last = steps - 1;
    // Workgroup i starts four i steps (128 bytes) into its K range and wraps around: started together, all
    // workgroups ask for the same bytes of rows 2 K bytes apart at once, which fall on a fraction of the
    // memory channels (3-8 % on weights of 8192 to 128256 rows).
    const int first = (int)(((uint32_t)blockIdx.x * 4u) % (uint32_t)steps);
    constexpr int D = kDenseDepth;
    uint4_t bq[D][NT], aq[D][MT];
    auto load = [&](int slot, int s) {
        int at = min(s, last) + first;
        if (at >= steps) at -= steps;
        const size_t off = (size_t)at * 32;
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
    if constexpr (KS > 1) {
        __shared__ float4_t sums[KS - 1][MT * NT][64];
        if (wave > 0) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) sums[wave - 1][mt * NT + nt][lane] = acc[mt][nt];
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int w = 0; w < KS - 1; ++w)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const float4_t v = sums[w][mt * NT + nt][lane];
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[mt][nt][r] += v[r];
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

// The waves of a workgroup share their columns and split K where the plain grid leaves CUs without a
// workgroup and every wave still keeps a full ring of steps.
static bool dense_share_k(unsigned workgroups, int K) {
    static const char* off = getenv("MH_F16_NO_SHARE_K");
    if (off && *off && atoi(off)) return false;
    return workgroups < (unsigned)compute_units() && K % 128 == 0 && K / 128 >= kDenseDepth;
}

// One to eight rows of a (decode): a dot-product kernel.  The MFMA kernel above reads b
// in 64-byte pieces of 16 rows per wave load and leaves most of the MFMA tile empty; here
// a wave streams whole rows of b, 1 KiB per load (lane l holds k = 512 i + 8 l .. + 8),
// four rows at a time, against a copy of a in LDS (one 16-byte LDS read per row of a
// serves the four rows of b), with two steps of loads in flight across the boundaries
// between row groups.  Products of fp16 pairs are added in fp32 (v_dot2_f32_f16), the
// 64 lanes' sums by shuffles.  K is a multiple of 1024; a wave owns a contiguous run of
// row groups.  Up to four rows of a: two workgroups of four waves per CU; five to eight
// rows (up to 128 KiB of LDS): one workgroup of eight waves.
constexpr int kGemvRows = 4;  // rows of b per wave and step

template <int MR>
__global__ __launch_bounds__(512) void f16_gemv_nk_kernel(const half_t* __restrict__ a, const half_t* __restrict__ b,
                                                          half_t* __restrict__ out, int M, int N, int K) {
    extern __shared__ uint4_t gemv_xs[];  // [MR][K / 8]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wg_waves = blockDim.x >> 6;
    const int k8 = K / 8;
    for (int i = tid; i < MR * k8; i += blockDim.x) {
        const int m = min(i / k8, M - 1);
        gemv_xs[i] = *reinterpret_cast<const uint4_t*>(a + (size_t)m * K + (size_t)(i % k8) * 8);
    }
    __syncthreads();

    // row groups of this wave: the first `extra` waves of the grid take one more
    const int groups = (N + kGemvRows - 1) / kGemvRows, waves = gridDim.x * wg_waves, w = blockIdx.x * wg_waves + wave;
    const int share = groups / waves, extra = groups % waves;
    const int first = w * share + min(w, extra), count = share + (w < extra ? 1 : 0);
    if (count == 0) return;
    const int kc = K / 512;  // steps per row group (even)
    const int total = count * kc;

    // (group, step) of the next load, advanced in wave-uniform registers
    int lg = first, ls = 0, issued = 0;
    auto load = [&](uint4_t (&q)[kGemvRows]) {
#pragma unroll
        for (int r = 0; r < kGemvRows; ++r) {
            const int n = min(lg * kGemvRows + r, N - 1);
            q[r] = __builtin_nontemporal_load(
                reinterpret_cast<const uint4_t*>(b + (size_t)n * K + (size_t)ls * 512 + lane * 8));
        }
        if (++issued < total) {  // past the end the last step is read again and not used
            if (++ls == kc) {
                ls = 0;
                ++lg;
            }
        }
    };
    float acc[kGemvRows][MR];
    auto clear = [&]() {
#pragma unroll
        for (int r = 0; r < kGemvRows; ++r)
#pragma unroll
            for (int m = 0; m < MR; ++m) acc[r][m] = 0.f;
    };
    auto consume = [&](const uint4_t (&q)[kGemvRows], int step) {
#pragma unroll
        for (int m = 0; m < MR; ++m) {
            const uint4_t xv = gemv_xs[m * k8 + step * 64 + lane];
            const unsigned int xw[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
            for (int r = 0; r < kGemvRows; ++r) {
                const unsigned int bw[4] = {q[r].x, q[r].y, q[r].z, q[r].w};
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    acc[r][m] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, xw[e]),
                                                       __builtin_bit_cast(half2_t, bw[e]), acc[r][m], false);
            }
        }
    };
    auto finish = [&](int group) {
#pragma unroll
        for (int r = 0; r < kGemvRows; ++r)
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                const float v = wave_sum(acc[r][m]);
                const int n = group * kGemvRows + r;
                if (lane == 0 && m < M && n < N) out[(size_t)m * N + n] = (half_t)v;
            }
        clear();
    };

    uint4_t q0[kGemvRows], q1[kGemvRows];
    clear();
    load(q0);
    int group = first;
    for (int step = 0, done = 0; done < total; done += 2) {
        load(q1);
        consume(q0, step);
        load(q0);
        consume(q1, step + 1);
        step += 2;
        if (step == kc) {
            finish(group);
            step = 0;
            ++group;
            // two waves share a SIMD (of one workgroup of eight waves or of two of four) and the older
            // one is served first: the priority falls with the row groups a wave has behind it, so
            // that the younger one does not finish alone
            set_priority_by_progress(group - first, count);
        }
    }
}

// Any K (no divisibility or alignment assumptions): one thread per output.
__global__ void f16_matmul_nk_generic_kernel(const half_t* __restrict__ a, const half_t* __restrict__ b,
                                             half_t* __restrict__ out, int M, int N, int K) {
    a += (size_t)blockIdx.y * M * K;  // blockIdx.y: the matrix of a batch
    b += (size_t)blockIdx.y * N * K;
    out += (size_t)blockIdx.y * M * N;
    const size_t total = (size_t)M * N;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
        const int m = (int)(idx / N), n = (int)(idx % N);
        float acc = 0.f;
        for (int k = 0; k < K; ++k) acc = __builtin_fmaf((float)a[(size_t)m * K + k], (float)b[(size_t)n * K + k], acc);
        out[idx] = (half_t)acc;
    }
}

// The eight-row dot-product kernel takes more dynamic LDS than a launch may ask for by
// default: raised once per device.  Callers that record launches into a graph call this
// beforehand (mh_llama_create does), so that no attribute call falls into a recording.
int f16_gemv_prepare() {
    static bool done[64] = {};
    int dev = 0;
    MH_CHECK_HIP(hipGetDevice(&dev));
    if (dev >= 0 && dev < 64 && done[dev]) return MH_OK;
    MH_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&f16_gemv_nk_kernel<8>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, 131072));
    if (dev >= 0 && dev < 64) done[dev] = true;
    return MH_OK;
}

}  // namespace mh

namespace mh {
// f16_matmul_lds.hip
bool f16_matmul_lds_supported(int M, int N, int K);
int f16_matmul_lds_launch(hipStream_t stream, const void* a, const void* b, void* out, int batch, int M, int N, int K);
}  // namespace mh

using namespace mh;

// The MFMA kernels for `batch` matrices (K a multiple of 32, every matrix on a 16-byte boundary): the weight
// streamed through LDS in whole lines where that kernel serves the shape, operands straight from global
// memory otherwise.  Kernel and tiling depend on M, N and K only.
static int launch_dense_mfma(hipStream_t st, const void* a, const void* b, void* out, int batch, int M, int N, int K) {
    if (f16_matmul_lds_supported(M, N, K) && (M + 63) / 64 <= 65535) return f16_matmul_lds_launch(st, a, b, out, batch, M, N, K);
    const int mt = M <= 16 ? 1 : M <= 32 ? 2 : 4;
    const int nt = mt == 1 ? 1 : 2;  // columns per wave: 16 or 32
    dim3 grid((N + 64 * nt - 1) / (64 * nt), (M + 16 * mt - 1) / (16 * mt), batch);
    MH_REQUIRE(grid.y <= 65535, "dense fp16 product: M=%d is too large for one launch", M);
    const bool share_k = dense_share_k(grid.x * grid.y, K);
    if (share_k) grid.x = (N + 16 * nt - 1) / (16 * nt);
#define MH_DENSE(MT, NT)                                                                                            \
    if (share_k)                                                                                                    \
        hipLaunchKernelGGL((f16_matmul_nk_kernel<MT, NT, 4>), grid, dim3(256), 0, st, (const half_t*)a,            \
                           (const half_t*)b, (half_t*)out, M, N, K);                                                \
    else                                                                                                            \
        hipLaunchKernelGGL((f16_matmul_nk_kernel<MT, NT, 1>), grid, dim3(256), 0, st, (const half_t*)a,            \
                           (const half_t*)b, (half_t*)out, M, N, K)
    switch (mt) {
        case 1: MH_DENSE(1, 1); break;
        case 2: MH_DENSE(2, 2); break;
        default: MH_DENSE(4, 2); break;
    }
#undef MH_DENSE
    MH_CHECK_LAUNCH();
    return MH_OK;
}

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
    // one to eight rows against a weight with at least one row group per wave: dot products
    static const char* no_gemv = getenv("MH_F16_NO_GEMV");
    const int mr = M == 1 ? 1 : M == 2 ? 2 : M <= 4 ? 4 : 8;
    const size_t lds = (size_t)mr * K * sizeof(half_t);
    if (M <= 8 && K % 1024 == 0 && lds <= (mr == 8 ? 131072u : 65536u) && N >= compute_units() * 8 * kGemvRows &&
        !(no_gemv && *no_gemv && atoi(no_gemv))) {
        // eight waves per CU either way
        const int wgs = mr == 8 ? compute_units() : compute_units() * 2, threads = mr == 8 ? 512 : 256;
#define MH_GEMV(MR)                                                                                              \
    hipLaunchKernelGGL((f16_gemv_nk_kernel<MR>), dim3(wgs), dim3(threads), lds, st, (const half_t*)a,             \
                       (const half_t*)b, (half_t*)out, M, N, K)
        switch (mr) {
            case 1: MH_GEMV(1); break;
            case 2: MH_GEMV(2); break;
            case 4: MH_GEMV(4); break;
            default: {
                const int rc = f16_gemv_prepare();
                if (rc) return rc;
                MH_GEMV(8);
                break;
            }
        }
#undef MH_GEMV
        MH_CHECK_LAUNCH();
        return MH_OK;
    }
    return launch_dense_mfma(st, a, b, out, 1, M, N, K);
}

// One launch for a batch of independent products: blockIdx.z (blockIdx.y of the generic kernel)
// walks the matrices, each with the tiling of a single product.
extern "C" int mh_f16_matmul_nk_batched(mh_stream_t stream, const void* a, const void* b, void* out, int batch,
                                        int M, int N, int K) {
    MH_REQUIRE(batch >= 0 && M >= 0 && N >= 0 && K >= 0, "mh_f16_matmul_nk_batched: bad shape batch=%d M=%d N=%d K=%d",
               batch, M, N, K);
    if (batch == 0 || M == 0 || N == 0) return MH_OK;
    if (batch == 1) return mh_f16_matmul_nk(stream, a, b, out, M, N, K);
    MH_REQUIRE(a && b && out, "mh_f16_matmul_nk_batched: null pointer");
    MH_REQUIRE(batch <= 65535, "mh_f16_matmul_nk_batched: at most 65535 matrices per call, got %d", batch);
    hipStream_t st = as_stream(stream);
    // every matrix of the batch must start on a 16-byte boundary for the vector loads
    const bool fast = K > 0 && K % 32 == 0 && ((uintptr_t)a | (uintptr_t)b) % 16 == 0 &&
                      ((size_t)M * K * 2) % 16 == 0 && ((size_t)N * K * 2) % 16 == 0;
    if (!fast) {
        size_t blocks = ((size_t)M * N + 255) / 256;
        const size_t cap = (size_t)compute_units() * 16;
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL(f16_matmul_nk_generic_kernel, dim3((unsigned)blocks, batch), dim3(256), 0, st,
                           (const half_t*)a, (const half_t*)b, (half_t*)out, M, N, K);
        MH_CHECK_LAUNCH();
        return MH_OK;
    }
    // the single product's choice of kernel and tiling: a matrix of a batch gets the bits it gets alone
    return launch_dense_mfma(st, a, b, out, batch, M, N, K);
}
