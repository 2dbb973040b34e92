// W8A8 int8 GEMM, operand tiles fetched straight from global memory into LDS.
//
// Block tile 128 x 256, 128-k stages, eight waves 2 x 4, each 64 x 64 as 4 x 4 tiles
// of v_mfma_i32_16x16x64_i8; a k-step is two 64-k halves with double-buffered
// fragments (lane l: 16 bytes of row l % 16, k chunk l / 16).  The 16 x 16 x 64 form
// is chosen for what the part sustains under its power limit: a register-resident
// stream of it on random int8 operands runs at 4.1 POP/s (2.06 GHz) where the
// 32 x 32 x 32 form runs at 3.3 POP/s (1.68 GHz), at the same fragment bytes per MAC.
// gfx950's 128-bit LDS-destination buffer loads write 16 bytes per lane to consecutive
// LDS addresses (wave base in M0), so there is no register ring, no ds_write and no
// wait for loaded registers on the issue path.  The LDS swizzle that keeps the
// fragment reads conflict-free is applied on the global side instead: a wave load
// covers eight 128-byte LDS rows, and the lane that fills chunk position c' of row r
// fetches chunk c' ^ ((r >> 1) & 7) of that row's line.  Without a ring's
// registers three stages fit into LDS (144 KiB), which lets a stage be requested
// almost three k-steps before its first use.
//
// Ordering: the loads are issued from inline assembly, so the compiler neither
// counts them nor knows that they write LDS; every wave waits for its own loads
// of a stage with an explicit s_waitcnt vmcnt before the barrier that publishes
// the stage, and for its own fragment reads of a buffer before the barrier after
// which the buffer is refilled.
#include "common.h"

namespace mh {

constexpr int kDmaBM = 128, kDmaBN = 256, kDmaBK = 128, kDmaThreads = 512, kDmaStages = 3;
constexpr int kDmaStageBytes = (kDmaBM + kDmaBN) * kDmaBK;  // 48 KiB
constexpr int kDmaLoads = kDmaStageBytes / 1024 / 8;        // wave loads per wave and stage: 6
constexpr int kDmaStagePitch = 144;                         // epilogue: 64 fp16 + 16 bytes of padding per row

// 16 bytes per lane, global -> LDS at m0 + lane * 16.  voffset: the lane's byte offset,
// soffset: the scalar (k) offset; out-of-range records read as zero.
__device__ __forceinline__ void load_to_lds(uint32_t lds_addr, int voffset, const int4_t& rsrc, int soffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset) : "memory", "m0");
}

__device__ __forceinline__ int4_t make_rsrc(const void* base, uint32_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    int4_t r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)((a >> 32) & 0xffffu));
    r[2] = __builtin_amdgcn_readfirstlane((int)bytes);
    r[3] = kBufferRsrcFlags;
    return r;
}

__global__ __launch_bounds__(kDmaThreads) void i8_gemm_dma_kernel(
    const int8_t* __restrict__ A, const int8_t* __restrict__ W, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, half_t* __restrict__ out, int32_t* __restrict__ acc_out,
    int M, int N, int K, int tiles_m, int tiles_n, int group_m, int xcd_chunk) {
    constexpr int BK = kDmaBK;
    // [3][A tile | W tile]; reused by the epilogue as eight 32-row output stages
    __shared__ __attribute__((aligned(1024))) int8_t smem[kDmaStages * kDmaStageBytes];
    auto As = [&](int buf) { return smem + buf * kDmaStageBytes; };
    auto Bs = [&](int buf) { return smem + buf * kDmaStageBytes + kDmaBM * BK; };

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
    const int m0 = tm * kDmaBM, n0 = tn * kDmaBN;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wy = wave >> 2, wx = wave & 3;
    const int l16 = lane & 15, lg = lane >> 4;

    // The scales of this lane's results (rows i * 16 + l16, columns j * 16 + lg * 4 .. + 3 of the wave
    // tile), requested here and used in the epilogue.  They stay in registers: staged through LDS at
    // this point, two loads, each waited for and stored, stood in front of the first operand load of
    // every launch (two memory round trips, 2 us of a 31 us launch).
    // (No branch around the loads -- the values of a branch are waited for where it ends: without an
    // fp16 output, when the scales may be absent, the loads read the first words of A instead.)
    float sa_r[4];
    float4_t sw_r[4];
    {
        const float* as = out ? a_scale : reinterpret_cast<const float*>(A);
        const float* ws = out ? w_scale : reinterpret_cast<const float*>(A);
        const int m_last = out ? M - 1 : 0, n_last = out ? N - 1 : 0;
        const int wm0 = m0 + (wave >> 2) * 64, wn0 = n0 + (wave & 3) * 64;
#pragma unroll
        for (int i = 0; i < 4; ++i) sa_r[i] = as[min(wm0 + i * 16 + l16, m_last)];
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) sw_r[j][e] = ws[min(wn0 + j * 16 + lg * 4 + e, n_last)];
    }

    int4_t acc[4][4];  // [m tile][n tile] of 16 x 16
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = int4_t{0, 0, 0, 0};

    // Wave load L = j * 8 + wave (j = 0..5) fills LDS rows L * 8 .. L * 8 + 7 of a stage:
    // rows 0..127 are the A tile (L < 16, j < 2), rows 128..383 the W tile.
    const int4_t a_rsrc = make_rsrc(A, (uint32_t)((size_t)M * K));
    const int4_t w_rsrc = make_rsrc(W, (uint32_t)((size_t)N * K));
    const int4_t none = make_rsrc(A, 0u);  // zero records: no traffic, zeros written
    int voff[kDmaLoads];
#pragma unroll
    for (int j = 0; j < kDmaLoads; ++j) {
        const int row = (j * 8 + wave) * 8 + (lane >> 3);             // row of the stage
        const int chunk = (lane & 7) ^ ((row >> 1) & 7);              // global chunk that lands at position lane & 7
        voff[j] = j < 2 ? min(m0 + row, M - 1) * K + chunk * 16 : min(n0 + row - kDmaBM, N - 1) * K + chunk * 16;
    }
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(size_t)smem) + (uint32_t)wave * 1024u;
    const int KT = K / BK;
    // part 0: the A rows and one W load, part 1: the other three W loads
    auto load_stage_piece = [&](int j, int stage) {
        const bool live = stage < KT;
        const uint32_t base = lds0 + (uint32_t)(stage % kDmaStages) * kDmaStageBytes;
        load_to_lds(base + (uint32_t)j * 8192u, voff[j], live ? (j < 2 ? a_rsrc : w_rsrc) : none, stage * BK);
    };
    auto load_stage_part = [&](int part, int stage) {
#pragma unroll
        for (int j = part * 3; j < part * 3 + 3; ++j) load_stage_piece(j, stage);
    };

    auto swz128 = [](int row, int chunk) { return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4); };
    // Fragments of one 64-k half of a stage: lane l holds 16 bytes of row l % 16, k chunk l / 16
    // (the same mapping for both operands, which is all a dot product needs).
    int4_t fa[2][4], fb[2][4];
    auto read_a = [&](int set, int buf, int half, int i) {
        fa[set][i] = *reinterpret_cast<const int4_t*>(As(buf) + swz128(wy * 64 + i * 16 + l16, half * 4 + lg));
    };
    auto read_b = [&](int set, int buf, int half, int j) {
        fb[set][j] = *reinterpret_cast<const int4_t*>(Bs(buf) + swz128(wx * 64 + j * 16 + l16, half * 4 + lg));
    };
    auto mfma_row = [&](int set, int i) {  // the four column tiles of row tile i
#pragma unroll
        for (int j = 0; j < 4; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[set][j], fa[set][i], acc[i][j], 0, 0, 0);
    };
    auto mfma_pair = [&](int set, int i, int j) {
        acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[set][j], fa[set][i], acc[i][j], 0, 0, 0);
        acc[i][j + 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[set][j + 1], fa[set][i], acc[i][j + 1], 0, 0, 0);
    };

    // Stage s lives in LDS buffer s % 3.  It is requested after the barrier of k-step
    // s - 3 (every wave has then read the last fragments of that buffer) and in the
    // first half of k-step s - 2, and must have landed at the barrier of k-step
    // s - 1, whose second half reads its first fragments.
#pragma unroll
    for (int s = 0; s < kDmaStages; ++s) {
        load_stage_part(0, s);
        load_stage_part(1, s);
    }
    asm volatile("s_waitcnt vmcnt(12)" ::: "memory");  // stage 0 of this wave
    __syncthreads();
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        read_a(0, 0, 0, t);
        read_b(0, 0, 0, t);
    }
    int buf = 0;
    for (int kt = 0; kt < KT; ++kt) {
        const int nbuf = buf == kDmaStages - 1 ? 0 : buf + 1;
        // first half: 16 MFMAs on set 0; the fragments of the second half and the second half of the
        // loads of stage kt + 2 go between them (one load between two pairs of MFMAs: issued back to
        // back by all eight waves the loads fill the vector memory queue and the waves stall in issue
        // with the matrix pipes idle)
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            mfma_pair(0, t >> 1, (t & 1) * 2);
            __builtin_amdgcn_sched_barrier(0);
            if (t < 4) {
                read_a(1, buf, 1, t);
                read_b(1, buf, 1, t);
            } else if (t < 7) {
                if (kt > 0) load_stage_piece(t - 1, kt + 2);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // second half, first quarter of its MFMAs
        mfma_row(1, 0);
        __builtin_amdgcn_sched_barrier(0);
        // stage kt + 1 of this wave has landed (the six loads of stage kt + 2 may still be
        // in flight) and this wave's reads of `buf` are complete: publish / release
        asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)" ::: "memory");
        __syncthreads();
        // the rest: first fragments of stage kt + 1 and the first half of the loads of stage kt + 3
        // into the buffer just released
#pragma unroll
        for (int t = 2; t < 8; ++t) {
            mfma_pair(1, t >> 1, (t & 1) * 2);
            __builtin_amdgcn_sched_barrier(0);
            if (t < 6) {
                read_a(0, nbuf, 0, t - 2);
                read_b(0, nbuf, 0, t - 2);
            }
            if (t >= 3 && t < 6) load_stage_piece(t - 3, kt + 3);
            __builtin_amdgcn_sched_barrier(0);
        }
        buf = nbuf;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the (empty) loads past the end write LDS too
    __syncthreads();  // every wave is done with the operand buffers

    // Epilogue.  acc[i][j][e] belongs to row m = i * 16 + l16 and column
    // n = j * 16 + lg * 4 + e of the wave tile: four consecutive n per lane.
    const int wm = wy * 64, wn = wx * 64;  // wave tile origin inside the block tile
    if (acc_out) {
        const bool n_vec = (N % 4 == 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = m0 + wm + i * 16 + l16;
            if (m >= M) continue;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = n0 + wn + j * 16 + lg * 4;
                if (n >= N) continue;
                int32_t* dst = acc_out + (size_t)m * N + n;
                if (n_vec && n + 4 <= N) {
                    *reinterpret_cast<int4_t*>(dst) = acc[i][j];
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < N) dst[e] = acc[i][j][e];
                }
            }
        }
    }
    if (out) {
        // Scaled fp16 values are staged per wave as 32 rows x 64 columns in LDS
        // and leave as whole 128-byte row pieces, 16 bytes per lane.
        int8_t* stage = smem + wave * (32 * kDmaStagePitch);
        const bool n_vec = (N % 8 == 0);
#pragma unroll
        for (int ip = 0; ip < 2; ++ip) {
#pragma unroll
            for (int ii = 0; ii < 2; ++ii) {
                const int i = ip * 2 + ii;
                const float sa = sa_r[i];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int nl = j * 16 + lg * 4;
                    const float4_t sw = sw_r[j];
                    half4_t h;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        // The scale product and its product with the sum are each rounded to
                        // fp32 and only then to fp16; the empty asm keeps the compiler from
                        // fusing the last two steps into one instruction that rounds once.
                        float prod = (float)acc[i][j][e] * (sa * sw[e]);
                        asm volatile("" : "+v"(prod));
                        h[e] = (half_t)prod;
                    }
                    *reinterpret_cast<half4_t*>(stage + (ii * 16 + l16) * kDmaStagePitch + nl * 2) = h;
                }
            }
            // wave-private region: only this wave's own LDS traffic has to land
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const int row = rr * 8 + (lane >> 3), c8 = (lane & 7) * 8;
                const int m = m0 + wm + ip * 32 + row, n = n0 + wn + c8;
                const int4_t v = *reinterpret_cast<const int4_t*>(stage + row * kDmaStagePitch + c8 * 2);
                if (m >= M || n >= N) continue;
                half_t* dst = out + (size_t)m * N + n;
                if (n_vec) {
                    // streamed out: with one tile per CU every workgroup stores at the same time, and the
                    // 16.8 MB of a 2048 x 4096 result are 3 us of the launch
                    __builtin_nontemporal_store(v, reinterpret_cast<int4_t*>(dst));
                } else {
                    const half_t* hv = reinterpret_cast<const half_t*>(&v);
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (n + e < N) dst[e] = hv[e];
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    }
}

// Host side: the caller (mh_i8_gemm) has checked the operands; this kernel needs
// K % 128 == 0, at least three k-steps and operands below 2 GiB (32-bit buffer offsets).
bool i8_gemm_dma_supported(int M, int N, int K) {
    static const char* off = getenv("MH_I8_NO_DMA");
    if (off && *off && atoi(off)) return false;
    return K % kDmaBK == 0 && K / kDmaBK >= kDmaStages && (size_t)M * K < ((size_t)1 << 31) &&
           (size_t)N * K < ((size_t)1 << 31);
}

int i8_gemm_dma_launch(hipStream_t stream, const int8_t* a, const int8_t* w, const float* a_scale,
                       const float* w_scale, void* out_f16, int32_t* acc_i32, int M, int N, int K) {
    const int tiles_m = (M + kDmaBM - 1) / kDmaBM, tiles_n = (N + kDmaBN - 1) / kDmaBN;
    const int tiles = tiles_m * tiles_n;
    const int group_m = tiles_m < 8 ? tiles_m : 8;
    const int xcd_chunk = (tiles % 8 == 0) ? tiles / 8 : 0;
    hipLaunchKernelGGL(i8_gemm_dma_kernel, dim3(tiles), dim3(kDmaThreads), 0, stream, a, w, a_scale, w_scale,
                       (half_t*)out_f16, acc_i32, M, N, K, tiles_m, tiles_n, group_m, xcd_chunk);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

}  // namespace mh
