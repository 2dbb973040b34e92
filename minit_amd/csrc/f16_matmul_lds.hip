// Dense fp16 product out[M, N] = a[M, K] @ b[N, K]^T for 9 to 64 rows per block against a long weight
// (the unquantized lm_head of the decode loop, 128256 x 8192, at batches above 8): the weight is
// streamed through LDS in whole 128-byte lines.
//
// Replaces the reference's library call for this shape (minit/cuda/dispatch.py:59-78,
// minit/cuda/kernel/cublas.py:68-111) where f16_matmul_nk_kernel loads its MFMA operands straight
// from global memory: there a wave load touches 64 bytes of 16 weight rows each (half a line per
// row) and the activations are re-read per 32 columns of a wave, 581-636 us for the lm_head at
// 16-32 rows against 308-366 us for the dot-product kernel at 1-8 rows.
//
// A workgroup of eight waves owns 128 weight rows (output columns) and up to 64 activation rows
// and walks K in rounds of 64 k = one 128-byte line of every row.  A stage is 128 + 64 rows of 128
// bytes (24 KiB), six stages in LDS; every wave fetches three 1 KiB pieces of a stage (eight rows
// x 128 bytes, two of the weight and one of the activations) with buffer_load_dwordx4 ... lds,
// five rounds ahead, 120 KiB in flight per CU.  The LDS side of such a load is lane-linear, so the
// XOR swizzle that keeps the operand reads (16 rows x one 16-byte chunk per quarter wave) free of
// bank conflicts is applied to the global address.  Wave w computes the 16 columns 16 w .. 16 w + 15
// for all row tiles: per round two B-operand reads, 2 MT A-operand reads and 2 MT MFMAs.  Rows of
// either operand past the end of its matrix are past the end of its buffer and read as zero.
//
// Measured, lm_head 128256 x 8192: 346-359 us at 9 to 64 rows (5.9-6.1 TB/s), flat in the row count,
// against 581-636 us before; 467-494 us while every workgroup started at k = 0 (see the start round
// below).  Rounds of 128 k (256-byte pieces, four stages of 40 KiB) measured slower then, 494 against
// 472 us at 32 rows.
#include "common.h"

namespace mh {

constexpr int kLdsBN = 128, kLdsBK = 64, kLdsStages = 6, kLdsThreads = 512;
constexpr int kLdsWBytes = kLdsBN * 128, kLdsXBytes = 64 * 128;
constexpr int kLdsStageBytes = kLdsWBytes + kLdsXBytes;

__device__ __forceinline__ int lds_swz(int row, int chunk) { return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4); }

__device__ __forceinline__ int4_t lds_rsrc(const void* base, uint32_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    int4_t r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)((a >> 32) & 0xffffu));
    r[2] = __builtin_amdgcn_readfirstlane((int)bytes);
    r[3] = kBufferRsrcFlags;
    return r;
}
// 16 bytes per lane, global -> LDS at m0 + lane * 16; out-of-range records write zeros.
__device__ __forceinline__ void lds_load(uint32_t lds_addr, int voffset, const int4_t& rsrc, int soffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset) : "memory", "m0");
}

// MT: 16-row tiles of activations per workgroup (2: up to 32 rows, 4: up to 64).
template <int MT>
__global__ __launch_bounds__(kLdsThreads) void f16_matmul_nk_lds_kernel(const half_t* __restrict__ a,
                                                                         const half_t* __restrict__ b,
                                                                         half_t* __restrict__ out, int M, int N, int K) {
    __shared__ __attribute__((aligned(1024))) int8_t smem[kLdsStages * kLdsStageBytes];
    // blockIdx.z: the matrix of a batch (a [batch, M, K], b [batch, N, K], out [batch, M, N])
    a += (size_t)blockIdx.z * M * K;
    b += (size_t)blockIdx.z * N * K;
    out += (size_t)blockIdx.z * M * N;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15, o = lane >> 4;
    const int n0 = blockIdx.x * kLdsBN, m0 = blockIdx.y * (16 * MT);
    const int rounds = K / kLdsBK;
    // Workgroup i starts i rounds into K and wraps around.  Started together, every CU of the chip asks for
    // the same 128 bytes of rows 2 K bytes apart at the same time, and for a K of some KiB those addresses
    // fall on a fraction of the memory channels: lm_head 128256 x 8192 at 32 rows 471-481 us started
    // together, 346-356 us staggered by one, seven or 37 rounds, 506-512 us staggered by 16 rounds (2 KiB).
    const int first = (int)(blockIdx.x % (uint32_t)rounds);

    const int4_t w_rsrc = lds_rsrc(b, (uint32_t)((size_t)N * K * 2));
    const int4_t x_rsrc = lds_rsrc(a, (uint32_t)((size_t)M * K * 2));
    const int4_t none = lds_rsrc(a, 0u);

    // the wave's three pieces of a stage: weight rows 16 w .. 16 w + 15 (two pieces of eight rows), activation
    // rows 8 w .. 8 w + 7; lane l lands at row l / 8 of its piece, chunk position l % 8, which holds the
    // chunk (l % 8) ^ swizzle(row)
    int off[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        const int row = (i < 2 ? wave * 16 + i * 8 : wave * 8) + (lane >> 3);
        const int chunk = (lane & 7) ^ ((row >> 1) & 7);
        off[i] = (int)(((uint32_t)((i < 2 ? n0 : m0) + row) * (uint32_t)K + (uint32_t)chunk * 8u) * 2u);
    }
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(size_t)smem);
    const uint32_t lds_w = lds0 + (uint32_t)wave * 2048u, lds_x = lds0 + kLdsWBytes + (uint32_t)wave * 1024u;
    auto issue_piece = [&](int i, int stage) {
        const uint32_t base = (uint32_t)(stage % kLdsStages) * kLdsStageBytes;
        const bool live = stage < rounds;
        int at = stage + first;
        if (at >= rounds) at -= rounds;
        if (i < 2)
            lds_load(lds_w + base + (uint32_t)i * 1024u, off[i], live ? w_rsrc : none, at * 128);
        else
            lds_load(lds_x + base, off[2], live ? x_rsrc : none, at * 128);
    };

    float4_t acc[MT];
#pragma unroll
    for (int rt = 0; rt < MT; ++rt) acc[rt] = float4_t{0.f, 0.f, 0.f, 0.f};

#pragma unroll
    for (int s = 0; s < kLdsStages - 1; ++s)
#pragma unroll
        for (int i = 0; i < 3; ++i) issue_piece(i, s);

    const int b_off = lds_swz(wave * 16 + j, o), a_off = kLdsWBytes + lds_swz(j, o);  // chunk o; + 64 bytes for the second k step
    for (int r = 0; r < rounds; ++r) {
        // stage r of this wave has landed; the three loads of each of the last four rounds may be in flight
        asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
        __syncthreads();
        // every wave has read stage r - 1: its buffer takes stage r + 5, one load between two MFMAs
        const int8_t* st = smem + (r % kLdsStages) * kLdsStageBytes;
        half8_t fb[2], fa[MT][2];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            fb[ks] = *reinterpret_cast<const half8_t*>(st + (b_off ^ (ks << 6)));
#pragma unroll
            for (int rt = 0; rt < MT; ++rt) fa[rt][ks] = *reinterpret_cast<const half8_t*>(st + (a_off ^ (ks << 6)) + rt * 2048);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int rt = 0; rt < MT; ++rt) {
            acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[rt][0], fb[0], acc[rt], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (rt < 3) issue_piece(rt, r + kLdsStages - 1);
            __builtin_amdgcn_sched_barrier(0);
            acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[rt][1], fb[1], acc[rt], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (MT == 2 && rt == 1) issue_piece(2, r + kLdsStages - 1);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the (empty) loads past the end write LDS too

    // acc[rt][e] is row rt*16 + o*4 + e, column 16 w + j of the tile
    const int n = n0 + wave * 16 + j;
    if (n < N) {
#pragma unroll
        for (int rt = 0; rt < MT; ++rt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int m = m0 + rt * 16 + o * 4 + e;
                if (m < M) out[(size_t)m * N + n] = (half_t)acc[rt][e];
            }
    }
}

// Shapes this kernel takes from mh_f16_matmul_nk: more rows than the dot-product kernel serves, whole
// 128-byte lines, 32-bit buffer offsets.
bool f16_matmul_lds_supported(int M, int N, int K) {
    static const char* off = getenv("MH_F16_NO_LDS");
    if (off && *off && atoi(off)) return false;
    // up to 16 rows against a weight that leaves CUs without a tile, the kernel with MFMA operands straight from
    // global memory and K split over the waves is ahead (8192 x 8192 at 9 rows 35 us against 45, 4096 x 4096 at
    // 16 rows 13 against 18); from 17 rows this one is, whatever the number of tiles (1024 x 4096 at 32 rows 17.8
    // against 22.5, 8192 x 8192 at 64 / 256 / 1024 rows 57 / 57 / 209 against 72 / 206 / 843)
    const bool enough = M > 16 || N >= compute_units() * kLdsBN / 2;
    return M > 8 && K % kLdsBK == 0 && K >= kLdsBK * kLdsStages && enough &&
           (size_t)N * K * 2 + (size_t)kLdsBN * K * 2 < ((size_t)1 << 32) && (size_t)M * K * 2 < ((size_t)1 << 31);
}

int f16_matmul_lds_launch(hipStream_t stream, const void* a, const void* b, void* out, int batch, int M, int N, int K) {
    const int mt = M <= 32 ? 2 : 4;
    const dim3 grid((N + kLdsBN - 1) / kLdsBN, (M + 16 * mt - 1) / (16 * mt), batch);
    if (mt == 2)
        hipLaunchKernelGGL(f16_matmul_nk_lds_kernel<2>, grid, dim3(kLdsThreads), 0, stream, (const half_t*)a,
                           (const half_t*)b, (half_t*)out, M, N, K);
    else
        hipLaunchKernelGGL(f16_matmul_nk_lds_kernel<4>, grid, dim3(kLdsThreads), 0, stream, (const half_t*)a,
                           (const half_t*)b, (half_t*)out, M, N, K);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

}  // namespace mh
