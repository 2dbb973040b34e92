// GPTQ w4a16 / w8a16 dequant-GEMV for decode (M <= 4), wave64 VALU, no MFMA.
//
// Replaces the fused qmm kernel of the reference
// (examples/qwen1_5_int8.py:156-216) for small M without the matrix cores.
//
//   * qweight [K/P, N] is N-contiguous, so lanes walk N: a lane owns four
//     adjacent columns and fetches them with one 16-byte non-temporal load per
//     packed row; a wave streams 1 KiB-contiguous row segments, eight rows in
//     flight.
//   * the activations of the block's K range are staged once in LDS in the
//     k-order the extraction produces and read back as wave-uniform
//     broadcasts; each dequantised fp16 pair feeds one v_dot2_f32_f16 per
//     output row (17 VALU ops per packed word at M = 1).
//   * K is split over the four waves of a block (LDS), over blockIdx.y (fp32
//     partials summed in split order by a second tiny kernel: deterministic, no
//     atomics, no fences) and within a lane (private fp32 accumulators).
//   * zero points and scales are fetched once per (group, column) and folded
//     into packed fp16 constants (gptq_common.h).
//
// The MFMA kernel in gptq_gemm.hip needs 13 VALU ops per word and is what
// mh_gptq_matmul dispatches to by default; this kernel stays callable as
// mh_gptq_gemv and through MH_GEMV_MAX_M.
#include "gptq_common.h"

namespace mh {

#pragma clang fp contract(off)

constexpr int kGemvCols = 256;     // columns per block: 64 lanes x 4
constexpr int kGemvWaves = 4;      // waves per block, splitting K

template <int BITS, int M, int ROWS>
__global__ __launch_bounds__(256) void gptq_gemv_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ qweight,
    const uint32_t* __restrict__ qzeros, const half_t* __restrict__ scales,
    half_t* __restrict__ out, float* __restrict__ partial,
    int N, int K, int rows_per_group, int steps_total, int steps_per_wave, int split_k) {
    constexpr int P = Packing<BITS>::kPerWord;
    constexpr int PAIRS = Packing<BITS>::kPairs;
    constexpr uint32_t MASK = Packing<BITS>::kMask;

    // activations of this block's K range, in pair order: [M][rows_blk * PAIRS] words
    extern __shared__ uint32_t xs[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tile = blockIdx.x;
    const int split = blockIdx.y;
    const int n = tile * kGemvCols + lane * 4;
    const bool active = n < N;
    const int nc = active ? n : 0;

    const int rows_total = steps_total * ROWS;
    const int rows_blk = kGemvWaves * steps_per_wave * ROWS;
    const int row_base = split * rows_blk;
    const int slot = split * kGemvWaves + wave;
    const int step_begin = slot * steps_per_wave;
    const int step_end = min(steps_total, step_begin + steps_per_wave);

    // The first step's weight rows are requested before anything else, so that
    // staging the activations overlaps their latency.
    uint4_t q[ROWS];
    auto load_rows = [&](int step) {
        const uint32_t* wp = qweight + (size_t)step * ROWS * N + nc;
#pragma unroll
        for (int i = 0; i < ROWS; ++i)
            q[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(wp + (size_t)i * N));
    };
    if (step_begin < step_end) load_rows(step_begin);

    for (int idx = threadIdx.x; idx < rows_blk * M; idx += 256) {
        const int m = idx / rows_blk, rl = idx % rows_blk;
        const int row = row_base + rl;
        uint32_t xv[PAIRS], xp[PAIRS];
#pragma unroll
        for (int p = 0; p < PAIRS; ++p) xv[p] = 0;
        if (row < rows_total) {
            const uint32_t* xr = reinterpret_cast<const uint32_t*>(x + (size_t)m * K + (size_t)row * P);
#pragma unroll
            for (int p = 0; p < PAIRS; ++p) xv[p] = xr[p];
        }
        pair_activations<BITS>(xv, xp);
#pragma unroll
        for (int p = 0; p < PAIRS; ++p) xs[(m * rows_blk + rl) * PAIRS + p] = xp[p];
    }
    __syncthreads();

    DequantRegs regs;
    regs.init(BITS);

    float acc[M][4];
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[m][c] = 0.f;

    ColumnConst cc[4];
    int g_cur = -1;
    for (int step = step_begin; step < step_end; ++step) {
        const int row = step * ROWS;
        if (step != step_begin) load_rows(step);
        const int g = row / rows_per_group;
        if (g != g_cur) {
            g_cur = g;
            const uint2 sraw = *reinterpret_cast<const uint2*>(scales + (size_t)g * N + nc);
            const uint32_t zword = qzeros[(size_t)g * (N / P) + nc / P] >> ((nc % P) * BITS);
            const half2_t s01 = as_half2(sraw.x), s23 = as_half2(sraw.y);
            cc[0] = make_column_const(s01.x, zword & MASK);
            cc[1] = make_column_const(s01.y, (zword >> BITS) & MASK);
            cc[2] = make_column_const(s23.x, (zword >> (2 * BITS)) & MASK);
            cc[3] = make_column_const(s23.y, (zword >> (3 * BITS)) & MASK);
        }
        const int rl0 = row - row_base;
#pragma unroll
        for (int i = 0; i < ROWS; ++i) {
            uint32_t xp[M][PAIRS];
#pragma unroll
            for (int m = 0; m < M; ++m)
#pragma unroll
                for (int p = 0; p < PAIRS; ++p) xp[m][p] = xs[(m * rows_blk + rl0 + i) * PAIRS + p];
            const uint32_t qs[4] = {q[i].x, q[i].y, q[i].z, q[i].w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                half2_t w[PAIRS];
                dequant_word<BITS>(qs[c], cc[c], regs, w);
#pragma unroll
                for (int m = 0; m < M; ++m)
#pragma unroll
                    for (int p = 0; p < PAIRS; ++p)
                        acc[m][c] = __builtin_amdgcn_fdot2(as_half2(xp[m][p]), w[p], acc[m][c], false);
            }
        }
    }

    // K-reduction across the four waves of the block.
    __shared__ float red[kGemvWaves][M][kGemvCols];
#pragma unroll
    for (int m = 0; m < M; ++m)
        *reinterpret_cast<float4*>(&red[wave][m][lane * 4]) =
            make_float4(acc[m][0], acc[m][1], acc[m][2], acc[m][3]);
    __syncthreads();

    const int t = threadIdx.x;
    const int nt = tile * kGemvCols + t;
    if (nt >= N) return;
#pragma unroll
    for (int m = 0; m < M; ++m) {
        const float total = (red[0][m][t] + red[1][m][t]) + (red[2][m][t] + red[3][m][t]);
        if (split_k == 1)
            out[(size_t)m * N + nt] = (half_t)total;
        else
            partial[((size_t)split * M + m) * N + nt] = total;  // summed by splitk_finalize_kernel
    }
}

// Sum over the splits in split order with eight loads in flight: a loop that loads and adds per
// iteration is one memory round trip per split (16 splits: 6 of a 7.5 us launch).
__device__ __forceinline__ float4_t sum_splits_in_order(const float* __restrict__ p, size_t mn, int split_k) {
    float4_t s = {0.f, 0.f, 0.f, 0.f};
    for (int sp = 0; sp < split_k; sp += 8) {
        float4_t v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)  // past the last split: that split again (a cache hit), not added
            v[u] = *reinterpret_cast<const float4_t*>(p + (size_t)min(sp + u, split_k - 1) * mn);
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (sp + u < split_k) s += v[u];
    }
    return s;
}

// Second stage of split-K for the kernels that do not reduce in place:
// out[i] = fp16(sum over splits, in split order).  The kernel boundary makes
// the partials visible without any device-scope fence or atomic.
__global__ __launch_bounds__(256) void splitk_finalize_kernel(const float* __restrict__ partial,
                                                              half_t* __restrict__ out, size_t mn, int split_k,
                                                              const half_t* __restrict__ bias, int N) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= mn) return;
    const float4_t s = sum_splits_in_order(partial + i, mn, split_k);
    half4_t h = {(half_t)s[0], (half_t)s[1], (half_t)s[2], (half_t)s[3]};
    if (bias) h = h + *reinterpret_cast<const half4_t*>(bias + i % N);  // N % 8 == 0: four columns of one row
    *reinterpret_cast<half4_t*>(out + i) = h;
}

// The same with the SiLU-pair epilogue: out is [M, N / 2].
__global__ __launch_bounds__(256) void splitk_finalize_silu_kernel(const float* __restrict__ partial,
                                                                   half_t* __restrict__ out, int M, int N,
                                                                   int split_k, const half_t* __restrict__ bias) {
    const size_t half_n = (size_t)N / 2;
    const size_t o = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (o >= (size_t)M * half_n) return;
    const size_t m = o / half_n, j = o % half_n;
    const size_t gate = m * N + j / 128 * 256 + j % 128;
    const size_t mn = (size_t)M * N;
    const float4_t g = sum_splits_in_order(partial + gate, mn, split_k);
    const float4_t u = sum_splits_in_order(partial + gate + 128, mn, split_k);
    half4_t gh = {(half_t)g[0], (half_t)g[1], (half_t)g[2], (half_t)g[3]};
    half4_t uh = {(half_t)u[0], (half_t)u[1], (half_t)u[2], (half_t)u[3]};
    if (bias) {  // column of the gate sum within its row: gate - m * N
        gh = gh + *reinterpret_cast<const half4_t*>(bias + (gate - m * N));
        uh = uh + *reinterpret_cast<const half4_t*>(bias + (gate - m * N) + 128);
    }
    half4_t h;
#pragma unroll
    for (int e = 0; e < 4; ++e) h[e] = silu_pair(gh[e], uh[e]);
    *reinterpret_cast<half4_t*>(out + o) = h;
}

// kEpilogueResidual in the second stage: a workgroup covers 1024 consecutive
// columns of one row (N is a multiple of 1024), adds into the residual stream
// and leaves that piece's sum of squares in ssq_out[m, N / 1024].
__global__ __launch_bounds__(256) void splitk_finalize_residual_kernel(const float* __restrict__ partial, half_t* h,
                                                                       SmallFuse fuse, int M, int N, int split_k) {
    __shared__ float smem[16];
    const size_t mn = (size_t)M * N;
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;  // within one row: N % 1024 == 0
    // the old value of the stream, the next norm's weight and the bias are requested ahead of the
    // partial sums, whose wait then covers them
    const half4_t zero4 = {(half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f};
    const half4_t h_old = *reinterpret_cast<const half4_t*>(h + i);
    const half4_t nw = fuse.xw_out ? *reinterpret_cast<const half4_t*>(fuse.next_norm_w + i % N) : zero4;
    const half4_t b4 = fuse.bias ? *reinterpret_cast<const half4_t*>(fuse.bias + i % N) : zero4;
    const float4_t s = sum_splits_in_order(partial + i, mn, split_k);
    half4_t y = {(half_t)s[0], (half_t)s[1], (half_t)s[2], (half_t)s[3]};
    if (fuse.bias) y = y + b4;
    const half4_t r = h_old + y;  // fp16 add, one rounding
    *reinterpret_cast<half4_t*>(h + i) = r;
    if (fuse.xw_out) *reinterpret_cast<half4_t*>(fuse.xw_out + i) = norm_weighted(r, nw, fuse.xw_clamped);
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) ss += (float)r[e] * (float)r[e];
    ss = block_sum(ss, smem);
    if (threadIdx.x == 0) fuse.ssq_out[blockIdx.x] = ss;  // blocks are numbered row-major over [M, N / 1024]
}

// kEpilogueRopeAppend in the second stage: four consecutive columns = two
// interleaved pairs of one head.
__global__ __launch_bounds__(256) void splitk_finalize_rope_kernel(const float* __restrict__ partial, SmallFuse fuse,
                                                                   int M, int N, int split_k) {
    const size_t mn = (size_t)M * N;
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= mn) return;
    const int m = (int)(i / N), c = (int)(i % N);
    // the row's position is requested ahead of the partial sums (its cos / sin hang on it)
    const int pos = min(max(fuse.positions[m], 0), fuse.max_seq - 1);
    const float4_t sum = sum_splits_in_order(partial + i, mn, split_k);
    half4_t y = {(half_t)sum[0], (half_t)sum[1], (half_t)sum[2], (half_t)sum[3]};
    if (fuse.bias) y = y + *reinterpret_cast<const half4_t*>(fuse.bias + c);
    const int head = c / 128, d = c % 128;
    if (head >= fuse.q_heads + fuse.kv_heads) {  // value head: copied, cache is tiled
        half_t* dst = fuse.vt_cache + ((size_t)m * fuse.kv_heads + (head - fuse.q_heads - fuse.kv_heads)) * 128 * fuse.max_seq +
                      vt_offset(d, pos);
#pragma unroll
        for (int e = 0; e < 4; ++e) dst[e * kVTile] = y[e];
        return;
    }
    const float* cr = fuse.rope_cos + (size_t)pos * 64 + d / 2;
    const float* sr = fuse.rope_sin + (size_t)pos * 64 + d / 2;
    half4_t o;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const float re = (float)y[2 * j], im = (float)y[2 * j + 1];
        o[2 * j] = (half_t)(re * cr[j] - im * sr[j]);
        o[2 * j + 1] = (half_t)(im * cr[j] + re * sr[j]);
    }
    half_t* dst = head < fuse.q_heads
                      ? fuse.q_out + ((size_t)m * fuse.q_heads + head) * 128 + d
                      : fuse.k_cache + (((size_t)m * fuse.kv_heads + (head - fuse.q_heads)) * fuse.max_seq + pos) * 128 + d;
    *reinterpret_cast<half4_t*>(dst) = o;
}

void launch_splitk_finalize(hipStream_t stream, const float* partial, void* out, int M, int N, int split_k,
                            int epilogue, const SmallFuse& fuse) {
    if (epilogue == kEpilogueResidual) {
        hipLaunchKernelGGL(splitk_finalize_residual_kernel, dim3((unsigned)((size_t)M * N / 1024)), dim3(256), 0, stream,
                           partial, (half_t*)out, fuse, M, N, split_k);
        return;
    }
    if (epilogue == kEpilogueRopeAppend) {
        const size_t threads = ((size_t)M * N + 3) / 4;
        hipLaunchKernelGGL(splitk_finalize_rope_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream,
                           partial, fuse, M, N, split_k);
        return;
    }
    if (epilogue == kEpilogueSiluPairs) {
        const size_t threads = ((size_t)M * (N / 2) + 3) / 4;
        hipLaunchKernelGGL(splitk_finalize_silu_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0,
                           stream, partial, (half_t*)out, M, N, split_k, fuse.bias);
        return;
    }
    const size_t mn = (size_t)M * N;
    const size_t threads = (mn + 3) / 4;
    hipLaunchKernelGGL(splitk_finalize_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream,
                       partial, (half_t*)out, mn, split_k, fuse.bias, N);
}

// ---- host side -----------------------------------------------------------------------

struct GemvPlan {
    int rows;            // packed rows per step (template ROWS)
    int col_tiles;
    int split_k;
    int steps_total;
    int steps_per_wave;
};

static int env_int(const char* name, int fallback) {
    const char* v = getenv(name);
    if (!v || !*v) return fallback;
    return atoi(v);
}

GemvPlan plan_gemv(int N, int K, int group_size, int bits) {
    const int P = 32 / bits;
    const int rows_per_group = group_size / P;
    GemvPlan p;
    p.rows = (rows_per_group % 8 == 0) ? 8 : (rows_per_group % 4 == 0) ? 4 : 1;
    static const int rows_override = env_int("MH_GEMV_ROWS", 0);
    if (rows_override == 4 && p.rows == 8) p.rows = 4;
    p.col_tiles = (N + kGemvCols - 1) / kGemvCols;
    p.steps_total = (K / P) / p.rows;
    // Enough waves to keep every SIMD busy with several loads in flight.
    static const int waves_per_cu = env_int("MH_GEMV_WAVES_PER_CU", 16);
    const long target_waves = (long)compute_units() * waves_per_cu;
    long split = target_waves / ((long)p.col_tiles * kGemvWaves);
    const long max_split = (p.steps_total + kGemvWaves - 1) / kGemvWaves;
    // a block stages the activations of its K range in LDS: at most 512 packed rows
    const long max_steps_per_wave = 512 / (kGemvWaves * p.rows);
    const long min_split = (p.steps_total + kGemvWaves * max_steps_per_wave - 1) / (kGemvWaves * max_steps_per_wave);
    if (split > max_split) split = max_split;
    if (split < min_split) split = min_split;
    if (split < 1) split = 1;
    p.steps_per_wave = (int)((p.steps_total + split * kGemvWaves - 1) / (split * kGemvWaves));
    p.split_k = (p.steps_total + p.steps_per_wave * kGemvWaves - 1) / (p.steps_per_wave * kGemvWaves);
    return p;
}

size_t gemv_workspace_bytes(int M, int N, int K, int group_size, int bits) {
    const GemvPlan p = plan_gemv(N, K, group_size, bits);
    return (p.split_k > 1) ? kTileCounterBytes + (size_t)p.split_k * M * N * sizeof(float) : 0;
}

template <int BITS, int M, int ROWS>
static void launch_gemv(hipStream_t stream, const GemvPlan& p, const void* x, const int32_t* qweight,
                        const int32_t* qzeros, const void* scales, void* out, void* workspace,
                        int N, int K, int group_size) {
    constexpr int P = Packing<BITS>::kPerWord;
    // the head of the workspace holds the arrival counters of the MFMA kernel and stays zero
    float* partial = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + kTileCounterBytes);
    const size_t lds = (size_t)M * kGemvWaves * p.steps_per_wave * ROWS * Packing<BITS>::kPairs * sizeof(uint32_t);
    hipLaunchKernelGGL((gptq_gemv_kernel<BITS, M, ROWS>), dim3(p.col_tiles, p.split_k), dim3(256), lds, stream,
                       (const half_t*)x, (const uint32_t*)qweight, (const uint32_t*)qzeros,
                       (const half_t*)scales, (half_t*)out, partial, N, K, group_size / P,
                       p.steps_total, p.steps_per_wave, p.split_k);
    if (p.split_k > 1) launch_splitk_finalize(stream, partial, out, M, N, p.split_k, kEpilogueNone, SmallFuse{});
}

template <int BITS, int M>
static void launch_gemv_rows(hipStream_t stream, const GemvPlan& p, const void* x, const int32_t* qweight,
                             const int32_t* qzeros, const void* scales, void* out, void* workspace,
                             int N, int K, int group_size) {
    switch (p.rows) {
        case 8: launch_gemv<BITS, M, 8>(stream, p, x, qweight, qzeros, scales, out, workspace, N, K, group_size); break;
        case 4: launch_gemv<BITS, M, 4>(stream, p, x, qweight, qzeros, scales, out, workspace, N, K, group_size); break;
        default: launch_gemv<BITS, M, 1>(stream, p, x, qweight, qzeros, scales, out, workspace, N, K, group_size); break;
    }
}

template <int BITS>
static void launch_gemv_m(hipStream_t stream, const GemvPlan& p, const void* x, const int32_t* qweight,
                          const int32_t* qzeros, const void* scales, void* out, void* workspace,
                          int M, int N, int K, int group_size) {
    switch (M) {
        case 1: launch_gemv_rows<BITS, 1>(stream, p, x, qweight, qzeros, scales, out, workspace, N, K, group_size); break;
        case 2: launch_gemv_rows<BITS, 2>(stream, p, x, qweight, qzeros, scales, out, workspace, N, K, group_size); break;
        case 3: launch_gemv_rows<BITS, 3>(stream, p, x, qweight, qzeros, scales, out, workspace, N, K, group_size); break;
        default: launch_gemv_rows<BITS, 4>(stream, p, x, qweight, qzeros, scales, out, workspace, N, K, group_size); break;
    }
}

// Fast-path shape contract beyond check_gptq_args.
bool gemv_supported(int M, int N, int K, int group_size, int bits) {
    const int P = 32 / bits;
    return M >= 1 && M <= MH_GPTQ_GEMV_MAX_M && (bits == 4 || bits == 8) && group_size % P == 0 &&
           K % group_size == 0 && N % 8 == 0;
}

int gptq_gemv_launch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                     const void* scales, void* out, int M, int N, int K, int group_size, int bits,
                     void* workspace, size_t workspace_bytes) {
    const GemvPlan p = plan_gemv(N, K, group_size, bits);
    const size_t need = gemv_workspace_bytes(M, N, K, group_size, bits);
    if (p.split_k > 1) {
        if (workspace == nullptr || workspace_bytes < need)
            return fail(MH_ERR_WORKSPACE, "mh_gptq_gemv: workspace of %zu bytes required, got %zu", need,
                        workspace ? workspace_bytes : (size_t)0);
        if ((uintptr_t)workspace % 256 != 0)
            return fail(MH_ERR_WORKSPACE, "mh_gptq_gemv: workspace must be 256-byte aligned");
    }
    if (bits == 4)
        launch_gemv_m<4>(stream, p, x, qweight, qzeros, scales, out, workspace, M, N, K, group_size);
    else
        launch_gemv_m<8>(stream, p, x, qweight, qzeros, scales, out, workspace, M, N, K, group_size);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

}  // namespace mh
