// GPTQ w4a16 product for many rows (several hundred): dequantised fp16 weight tiles staged in
// LDS feed v_mfma_f32_16x16x32_f16.
//
// Replaces the same reference pair as the other product kernels
// (minit/quantize/dispatch.py:8-11 = Dequantize, then MatrixMultiply), in the regime
// where the arithmetic intensity (4 M flop per packed byte) is past the machine's
// ridge: a packed word must then be dequantised once per workgroup and shared by all
// of its rows, not once per wave or per block of 64 rows.
//
// Block tile 128 rows x 128 columns, 64 k per stage, four waves 2 x 2, each computing
// 64 x 64 as 4 x 4 MFMA tiles over two 32-k halves.  Per stage a thread
//   * fetches 64 bytes of activations (global -> registers two stages ahead -> LDS),
//   * fetches four packed words of one column = 32 k (global -> registers two stages
//     ahead), dequantises them with the same 13 instructions per word as every other
//     kernel here (W bit-identical to Dequantize), puts the pairs back into k order and
//     writes four 16-byte chunks into the column's row of the weight tile,
// while the MFMAs of the current stage run from the other LDS buffer.  Both tiles are
// stored as rows of 128 bytes (64 k of one activation row / one weight column) with
// the 16-byte chunk index XOR-ed with bits 1..3 of the row, which keeps the fragment
// reads (16 rows x one chunk per quarter wave) free of bank conflicts.  64 KiB of LDS
// and at most 128 registers: two workgroups per CU, two waves per SIMD.
//
// K is split over blockIdx.z when the tiles alone do not fill the chip; fp32 partial
// sums are added in split order by splitk_finalize_kernel (fixed order, repeatable).
#include "gptq_common.h"

#include <type_traits>

namespace mh {

constexpr int kWideBM = 128, kWideBN = 128, kWideBK = 64;
constexpr int kWideTileBytes = kWideBM * kWideBK * 2;  // 16 KiB: one operand tile of a stage

void launch_splitk_finalize(hipStream_t stream, const float* partial, void* out, int M, int N, int split_k,
                            int epilogue, const SmallFuse& fuse);

__device__ __forceinline__ int wide_swz(int row, int chunk) { return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4); }

// Loads issued from inline assembly: the compiler does not count them, so it inserts no waits of
// its own for them -- left to it, the wait at the loop header is for *every* outstanding load,
// which exposes the memory latency once per stage.  The kernel waits by hand (wide_wait) with the
// exact count, and hands the loaded registers through the wait so no use can move above it.
__device__ __forceinline__ int4_t wide_rsrc(const void* base, uint32_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    int4_t r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)((a >> 32) & 0xffffu));
    r[2] = __builtin_amdgcn_readfirstlane((int)bytes);
    r[3] = kBufferRsrcFlags;
    return r;
}
__device__ __forceinline__ void wide_load_b128(uint4_t& dst, int voffset, const int4_t& rsrc, int soffset) {
    asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(dst) : "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
}
__device__ __forceinline__ void wide_load_b32_stream(uint32_t& dst, int voffset, const int4_t& rsrc, int soffset) {
    asm volatile("buffer_load_dword %0, %1, %2, %3 offen sc1 nt" : "=v"(dst) : "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
}
__device__ __forceinline__ void wide_load_b32(uint32_t& dst, int voffset, const int4_t& rsrc, int soffset) {
    asm volatile("buffer_load_dword %0, %1, %2, %3 offen" : "=v"(dst) : "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
}
// Everything but the newest NEWEST loads has arrived; the registers that the next uses read pass
// through the wait, so that no use can be scheduled above it.
template <int NEWEST, int PT>
__device__ __forceinline__ void wide_wait(uint4_t (&a)[PT], uint32_t (&q)[PT], uint32_t& c0, uint32_t& c1) {
    if constexpr (PT == 4) {
        asm volatile("s_waitcnt vmcnt(%10)"
                     : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(q[0]), "+v"(q[1]), "+v"(q[2]), "+v"(q[3]),
                       "+v"(c0), "+v"(c1)
                     : "n"(NEWEST)
                     : "memory");
    } else {
        static_assert(PT == 2, "four or two pieces per thread");
        asm volatile("s_waitcnt vmcnt(%6)"
                     : "+v"(a[0]), "+v"(a[1]), "+v"(q[0]), "+v"(q[1]), "+v"(c0), "+v"(c1)
                     : "n"(NEWEST)
                     : "memory");
    }
}
__device__ __forceinline__ void wide_load_u16(uint32_t& dst, int voffset, const int4_t& rsrc, int soffset) {
    asm volatile("buffer_load_ushort %0, %1, %2, %3 offen" : "=v"(dst) : "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
}

// WN: waves along the columns of the tile.  WN = 2: four waves 2 x 2, 64 x 64 each (fewest fragment
// reads per MFMA; two workgroups per CU); WN = 4: eight waves 2 x 4, 64 x 32 each, for products of
// one or two row tiles, where the tiles are too few to give every SIMD two waves otherwise.
template <int WN>
__global__ __launch_bounds__(128 * WN, 2) void gptq_gemm_wide_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ qweight, const uint32_t* __restrict__ qzeros,
    const half_t* __restrict__ scales, half_t* __restrict__ out, float* __restrict__ partial, int M, int N, int K,
    int group_size, int stages_per_block, int split_k, const half_t* __restrict__ bias) {
    constexpr int T = 128 * WN;          // threads
    constexpr int PT = 1024 / T;         // per thread and stage: 16-byte chunks of activations = packed words
    constexpr int CT = 8 / WN;           // 16-column MFMA tiles per wave
    __shared__ __attribute__((aligned(16))) int8_t smem[2 * 2 * kWideTileBytes];  // [buffer][A | W]
    auto As = [&](int buf) { return smem + buf * 2 * kWideTileBytes; };
    auto Ws = [&](int buf) { return smem + buf * 2 * kWideTileBytes + kWideTileBytes; };

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wy = wave / WN, wx = wave % WN;
    const int nl = lane & 15, kq = lane >> 4;
    const int m0 = blockIdx.x * kWideBM, n0 = blockIdx.y * kWideBN;
    const int stages_total = K / kWideBK;
    const int s_begin = blockIdx.z * stages_per_block;
    const int n_stages = min(stages_per_block, stages_total - s_begin);

    // ---- what a thread fetches per stage
    // activations: chunk id j * T + tid of the 128 x 8 chunks of the tile
    int a_off[PT], a_lds[PT];
#pragma unroll
    for (int j = 0; j < PT; ++j) {
        const int id = j * T + tid, row = id >> 3, c = id & 7;
        a_off[j] = (min(m0 + row, M - 1) * K + c * 8) * 2;   // rows past M feed accumulator rows that are never stored
        a_lds[j] = wide_swz(row, c);
    }
    // weights: column tid % 128, PT consecutive packed rows of the stage's eight: 4-byte loads (a wave
    // load is 256 contiguous bytes of one packed row), and LDS writes in which sixteen consecutive
    // lanes hold sixteen consecutive columns at one chunk index -- the pattern of the fragment
    // reads, free of bank conflicts (a 16-byte load of four columns per thread makes every LDS
    // write a four-way conflict)
    const int w_prow = (tid >> 7) * PT, w_col = tid & 127;
    const bool w_live = n0 + w_col < N;
    const int w_cg = w_live ? n0 + w_col : 0;                  // a dead thread re-reads column 0 (never stored)
    const int4_t x_rsrc = wide_rsrc(x, (uint32_t)((size_t)M * K * 2));
    const int4_t q_rsrc = wide_rsrc(qweight, (uint32_t)((size_t)(K / 8) * N * 4));
    const int4_t s_rsrc = wide_rsrc(scales, (uint32_t)((size_t)(K / group_size) * N * 2));
    const int4_t z_rsrc = wide_rsrc(qzeros, (uint32_t)((size_t)(K / group_size) * (N / 8) * 4));
    int q_off[PT];
#pragma unroll
    for (int j = 0; j < PT; ++j) q_off[j] = ((w_prow + j) * N + w_cg) * 4;

    // 2 PT loads per stage, in this order
    uint4_t ra[2][PT];
    uint32_t rq[2][PT];
    auto fetch = [&](int slot, int stage) {
        const int s = min(stage, stages_total - 1);            // past the end: a repeat of the last stage, never used
#pragma unroll
        for (int j = 0; j < PT; ++j) wide_load_b128(ra[slot][j], a_off[j], x_rsrc, s * kWideBK * 2);
#pragma unroll
        for (int j = 0; j < PT; ++j) wide_load_b32_stream(rq[slot][j], q_off[j], q_rsrc, s * (kWideBK / 8) * N * 4);
    };

    // per-group constants of the thread's column
    DequantRegs regs;
    regs.init(4);
    ColumnConst cc;
    uint32_t raw_s, raw_z;
    const int last_group = K / group_size - 1;
    // two loads, in this order
    auto fetch_consts = [&](int group) {
        const int g = min(group, last_group);                   // past the end: never used
        wide_load_u16(raw_s, w_cg * 2, s_rsrc, g * N * 2);
        wide_load_b32(raw_z, (w_cg / 8) * 4, z_rsrc, g * (N / 8) * 4);
    };
    auto make_consts = [&]() {
        cc = make_column_const(__builtin_bit_cast(half_t, (uint16_t)raw_s), (raw_z >> ((w_cg & 7) * 4)) & 0xFu);
    };

    // registers -> LDS, one piece of a thread's share: a chunk of activations as it is, one packed
    // word dequantised into k order
    auto produce_piece = [&](int slot, int buf, int j) {
        *reinterpret_cast<uint4_t*>(As(buf) + a_lds[j]) = ra[slot][j];
        half2_t w[4];
        dequant_word<4>(rq[slot][j], cc, regs, w);              // (k0,k4) (k1,k5) (k2,k6) (k3,k7)
        const half2_t o0 = {w[0][0], w[1][0]}, o1 = {w[2][0], w[3][0]}, o2 = {w[0][1], w[1][1]}, o3 = {w[2][1], w[3][1]};
        const uint4_t packed = {as_u32(o0), as_u32(o1), as_u32(o2), as_u32(o3)};
        *reinterpret_cast<uint4_t*>(Ws(buf) + wide_swz(w_col, w_prow + j)) = packed;
    };

    float4_t acc[4][CT];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < CT; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

    // ---- pipeline: stage s is fetched during stage s - 2, written to LDS during stage s - 1
    const int spg = group_size / kWideBK;                       // stages per group (group_size is a multiple of 64)
    // (the constants travel like the weights: requested two stages ahead and with no branch around
    // the loads -- a conditional load makes the compiler wait for every outstanding load where the
    // branches meet, which would expose the memory latency once per stage)
    fetch(0, s_begin);
    fetch_consts(s_begin / spg);
    fetch(1, s_begin + 1);
    wide_wait<2 * PT, PT>(ra[0], rq[0], raw_s, raw_z);          // all but stage s_begin + 1
    make_consts();
    fetch_consts((s_begin + 1) / spg);
#pragma unroll
    for (int j = 0; j < PT; ++j) produce_piece(0, 0, j);
    fetch(0, s_begin + 2);
    __syncthreads();

    // one stage; PAR = parity of i, a compile-time value so that ring slots and LDS buffers are
    // fixed registers / addresses (a run-time slot index would turn the rings into indexed registers)
    auto run_stage = [&](auto par, int i) {
        constexpr int PAR = decltype(par)::value;
        const int stage = s_begin + i;
        // The order below is pinned with scheduling barriers: left alone, the compiler moves the
        // whole of the next stage's LDS writes in front of this stage's MFMAs.  First half: four
        // groups of MFMAs, the first PT of them followed by a piece of the next stage's production
        // (into the other buffer, which every wave left at the last barrier); the second half's
        // fragments are requested under the second group.  Second half: MFMAs only, the loads of
        // stage + 3 first.
        half8_t fa[2][4], fb[2][CT];
        auto read_frags = [&](int half) {
#pragma unroll
            for (int t = 0; t < 4; ++t)
                fa[half][t] = *reinterpret_cast<const half8_t*>(As(PAR) + wide_swz(wy * 64 + t * 16 + nl, half * 4 + kq));
#pragma unroll
            for (int t = 0; t < CT; ++t)
                fb[half][t] = *reinterpret_cast<const half8_t*>(Ws(PAR) + wide_swz((wx * CT + t) * 16 + nl, half * 4 + kq));
        };
        read_frags(0);
        // in flight at this point, oldest first: stage + 1 (other slot), the constants of its group,
        // stage + 2 (2 PT loads, may stay in flight)
        wide_wait<2 * PT, PT>(ra[PAR ^ 1], rq[PAR ^ 1], raw_s, raw_z);
        make_consts();                                          // of stage + 1
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
#pragma unroll
            for (int c = 0; c < CT; ++c)
                acc[r][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[0][r], fb[0][c], acc[r][c], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (r < PT) produce_piece(PAR ^ 1, PAR ^ 1, r);
            if (r == 1) read_frags(1);
            __builtin_amdgcn_sched_barrier(0);
        }
        fetch_consts((stage + 2) / spg);
        fetch(PAR ^ 1, stage + 3);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int c = 0; c < CT; ++c)
                acc[r][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[1][r], fb[1][c], acc[r][c], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
    };
    for (int i = 0; i < n_stages; i += 2) {
        run_stage(std::integral_constant<int, 0>{}, i);
        if (i + 1 < n_stages) run_stage(std::integral_constant<int, 1>{}, i + 1);
    }

    // the loads requested for stages past the end are still in flight: their registers are dead
    // to the compiler from here on, so let them land before anything else is put there
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    // ---- results: acc[r][c][e] is row wy*64 + r*16 + kq*4 + e, column (wx*CT + c)*16 + nl of the tile
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int m = m0 + wy * 64 + r * 16 + kq * 4 + e;
            if (m >= M) continue;
#pragma unroll
            for (int c = 0; c < CT; ++c) {
                const int n = n0 + (wx * CT + c) * 16 + nl;
                if (n >= N) continue;
                if (split_k == 1)
                    out[(size_t)m * N + n] = bias ? (half_t)acc[r][c][e] + bias[n] : (half_t)acc[r][c][e];
                else
                    partial[((size_t)blockIdx.z * M + m) * N + n] = acc[r][c][e];
            }
        }
}

// ---- host side ---------------------------------------------------------------------------

struct WidePlan {
    int tiles_m, tiles_n, split_k, stages_per_block;
};

static WidePlan plan_wide(int M, int N, int K) {
    WidePlan p;
    p.tiles_m = (M + kWideBM - 1) / kWideBM;
    p.tiles_n = (N + kWideBN - 1) / kWideBN;
    const int stages = K / kWideBK;
    const long tiles = (long)p.tiles_m * p.tiles_n;
    // two workgroups per CU fill the chip; a workgroup keeps at least eight stages, and the fp32
    // partial sums (8 M N bytes per split, written and read) stay below the packed weights' bytes
    long split = (2L * compute_units()) / tiles;
    if (split > stages / 8) split = stages / 8;
    const long traffic_cap = (long)K / (16L * M);
    if (split > traffic_cap) split = traffic_cap;
    if (split < 1) split = 1;
    p.stages_per_block = (int)((stages + split - 1) / split);
    p.split_k = (stages + p.stages_per_block - 1) / p.stages_per_block;
    return p;
}

bool gemm_wide_preferred(int M, int N, int K, int group_size, int bits, int epilogue) {
    static const char* off = getenv("MH_GEMM_NO_WIDE");
    if (off && *off && atoi(off)) return false;
    // measured against the 64-row blocks of the small-M kernel (us, this kernel / that one): 4096 x 14336 at
    // 192 rows 54.9 / 60.4, 256 rows 57.1 / 63.6, 512 rows 90.3 / 97.0, 2048 rows 315 / 336; 8192 x 28672 at 256
    // rows 159 / 173; 128 rows 39.4 / 37.7 (224 workgroups: one per CU, and split-K partial sums).  With few
    // tiles (14336 x 4096: 64 at 256 rows, 128 at 512) the long K walk of a tile needs a split whose fp32
    // partial sums cost more than the shared dequantisation saves (63.9 / 57.8 and, unsplit, 186 / 89), so
    // the tiles must cover three quarters of the CUs; MH_GEMM_WIDE_MIN_M moves the row switch
    static const int min_m = [] {
        const char* v = getenv("MH_GEMM_WIDE_MIN_M");
        return v && *v ? atoi(v) : 192;
    }();
    const long tiles = (long)((M + kWideBM - 1) / kWideBM) * ((N + kWideBN - 1) / kWideBN);
    return bits == 4 && epilogue == kEpilogueNone && M >= min_m && 4 * tiles >= 3L * compute_units() &&
           K % kWideBK == 0 && group_size % kWideBK == 0 && K % group_size == 0 && N % 8 == 0 &&
           (size_t)M * K * 2 < ((size_t)1 << 31) && (size_t)K * N / 2 < ((size_t)1 << 31);
}

size_t gemm_wide_workspace_bytes(int M, int N, int K) {
    const WidePlan p = plan_wide(M, N, K);
    return p.split_k > 1 ? kTileCounterBytes + (size_t)p.split_k * M * N * sizeof(float) : 0;
}

int gptq_gemm_wide_launch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                          const void* scales, void* out, int M, int N, int K, int group_size, void* workspace,
                          size_t workspace_bytes, const half_t* bias) {
    const WidePlan p = plan_wide(M, N, K);
    const size_t need = gemm_wide_workspace_bytes(M, N, K);
    if (need != 0 && (workspace == nullptr || workspace_bytes < need))
        return fail(MH_ERR_WORKSPACE, "mh_gptq_gemm: workspace of %zu bytes required, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    float* partial = need ? reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + kTileCounterBytes) : nullptr;
    // one or two row tiles: eight waves per workgroup, so that the few tiles still give every SIMD two waves
    if (p.tiles_m <= 2)
        hipLaunchKernelGGL(gptq_gemm_wide_kernel<4>, dim3(p.tiles_m, p.tiles_n, p.split_k), dim3(512), 0, stream,
                           (const half_t*)x, (const uint32_t*)qweight, (const uint32_t*)qzeros, (const half_t*)scales,
                           (half_t*)out, partial, M, N, K, group_size, p.stages_per_block, p.split_k, bias);
    else
        hipLaunchKernelGGL(gptq_gemm_wide_kernel<2>, dim3(p.tiles_m, p.tiles_n, p.split_k), dim3(256), 0, stream,
                           (const half_t*)x, (const uint32_t*)qweight, (const uint32_t*)qzeros, (const half_t*)scales,
                           (half_t*)out, partial, M, N, K, group_size, p.stages_per_block, p.split_k, bias);
    MH_CHECK_LAUNCH();
    if (p.split_k > 1) {
        SmallFuse fuse;
        fuse.bias = bias;
        launch_splitk_finalize(stream, partial, out, M, N, p.split_k, kEpilogueNone, fuse);
        MH_CHECK_LAUNCH();
    }
    return MH_OK;
}

}  // namespace mh
