// GPTQ w4a16 product for blocks of 128 (or 256) rows: weights dequantised in registers, straight into
// the B operand of v_mfma_f32_16x16x32_f16, activations fetched by LDS-destination loads.
//
// Replaces the same reference pair as the other product kernels
// (minit/quantize/dispatch.py:8-11 = Dequantize, then MatrixMultiply) above the small-M
// kernel (a packed word dequantised once per 64 rows, one wave per SIMD at these sizes).
//
// A workgroup of eight waves owns 128 rows x 128 columns over a K range, walked in rounds of
// 128 k.  Wave (cg, ks) owns all 128 rows x 64 columns (cg = 0, 1) and the ks-th 32 k of every
// round (ks = 0..3): 8 x 4 MFMA tiles, 128 accumulator registers, so a packed word is
// dequantised once for 128 rows and the 32 MFMAs of a 32-k step (512 cycles) outweigh its 84
// vector instructions.  (Blocks of 256 rows: four waves, one per SIMD, (cg, ks) with ks = 0, 1, rounds
// of 64 k, 16 x 4 tiles and 256 accumulators per wave, 64 MFMAs per step.)  Lane (j, o) of a
// wave holds columns 4j..4j+3 of the wave's 64 -- MFMA tile c takes column 4j + c -- and the
// o-th eight k of the step: its four packed words are one 16-byte load, its four scales one
// 8-byte load, its four zero points sit in one word.
//
// Per round every wave advances one step:
//   * all global loads are issued from inline assembly and waited for by hand; one
//     s_waitcnt vmcnt(14) per round covers everything the round consumes: the packed words and
//     constants of step r + 1 (requested four rounds ahead into a ring of four) and the
//     activation stage of round r (requested three rounds ahead into one of four 32 KiB LDS
//     buffers by buffer_load_dwordx4 ... lds: 128 rows x 256 bytes as two halves of 128-byte
//     rows; one load fills 1 KiB = eight rows of a half, whole 128-byte lines of the
//     activation matrix -- with 64-byte pieces every line crossed the L2-to-CU path twice and
//     the round took 1.35 us instead of the MFMAs' 0.62 -- and since the LDS side of such a
//     load is lane-linear, the XOR swizzle that keeps the A-operand reads (16 rows x one
//     16-byte chunk per quarter wave) free of bank conflicts is applied to the global address);
//   * one barrier;
//   * the 32 MFMAs of step r, with the round's seven loads and the dequantisation of step r + 1
//     (13 instructions per word = the bit-exact W of Dequantize, 4 to put the pairs back into k order, 4
//     for the column's constants) placed between them one or two instructions at a time
//     (kTallSchedule): two vector instructions per MFMA issue in its shadow, more cost 4.6 cycles each,
//     and one block of 17 behind every eighth MFMA left the matrix pipe idle.
// At the end the waves' shares of K are added through LDS in a fixed order (the waves that meet exchange
// halves of their accumulators, so that each ends up with its own share of the row tiles), the tile is
// turned into row-major order in LDS and leaves as 16-byte row pieces: fp16 results (plus bias), with
// kEpilogueSiluPairs silu(gate) * up of a tile made of 64 gate and the 64 matching up columns, or,
// with K split over blockIdx.y, fp32 partial sums for splitk_finalize_kernel.
#include "gptq_common.h"

#include <type_traits>

namespace mh {

constexpr int kTallBN = 128;
constexpr int kTallRoundK = 128;                 // K must be a multiple of this (four waves x one 32-k step)
// K shares (waves per column group) of a workgroup: four, or two where a wave owns sixteen row tiles and
// needs a SIMD's registers for itself
__host__ __device__ constexpr int tall_k_shares(int mt) { return mt == 16 ? 2 : 4; }

// A compile-time loop: f(integral_constant<int, S>) for S = BEGIN .. END - 1.
template <int BEGIN, int END, class F>
__device__ __forceinline__ void tall_static_for(F&& f) {
    if constexpr (BEGIN < END) {
        f(std::integral_constant<int, BEGIN>{});
        tall_static_for<BEGIN + 1, END>(f);
    }
}

void launch_splitk_finalize(hipStream_t stream, const float* partial, void* out, int M, int N, int split_k,
                            int epilogue, const SmallFuse& fuse);

__device__ __forceinline__ int tall_swz(int row, int chunk) { return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4); }

__device__ __forceinline__ int4_t tall_rsrc(const void* base, uint32_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    int4_t r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)((a >> 32) & 0xffffu));
    r[2] = __builtin_amdgcn_readfirstlane((int)bytes);
    r[3] = kBufferRsrcFlags;
    return r;
}
// Loads the compiler does not count (see the waits below); out-of-range records read as zero.
__device__ __forceinline__ void tall_load_b128_stream(uint4_t& dst, int voffset, const int4_t& rsrc, int soffset) {
    asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen sc1 nt" : "=v"(dst) : "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
}
__device__ __forceinline__ void tall_load_b64(uint2_t& dst, int voffset, const int4_t& rsrc, int soffset) {
    asm volatile("buffer_load_dwordx2 %0, %1, %2, %3 offen" : "=v"(dst) : "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
}
__device__ __forceinline__ void tall_load_b32(uint32_t& dst, int voffset, const int4_t& rsrc, int soffset) {
    asm volatile("buffer_load_dword %0, %1, %2, %3 offen" : "=v"(dst) : "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
}
// 16 bytes per lane, global -> LDS at m0 + lane * 16.
__device__ __forceinline__ void tall_load_to_lds(uint32_t lds_addr, int voffset, const int4_t& rsrc, int soffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset) : "memory", "m0");
}
// Two such loads behind one write of m0: the second lands 1 KiB further on in LDS through its instruction
// offset, which the global side adds as well (the caller's voffset1 is 1 KiB short).
__device__ __forceinline__ void tall_load_to_lds_pair(uint32_t lds_addr, int voffset0, int voffset1, const int4_t& rsrc, int soffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %3, %4 offen lds\n\t"
                 "buffer_load_dwordx4 %2, %3, %4 offen offset:1024 lds"
                 :: "s"(lds_addr), "v"(voffset0), "v"(voffset1), "s"(rsrc), "s"(soffset) : "memory", "m0");
}
// Everything but the newest NEWEST loads has arrived; the registers read next pass through the
// wait, so that no use can be scheduled above it.
template <int NEWEST>
__device__ __forceinline__ void tall_wait(uint4_t& q, uint2_t& s, uint32_t& z) {
    asm volatile("s_waitcnt vmcnt(%3)" : "+v"(q), "+v"(s), "+v"(z) : "n"(NEWEST) : "memory");
}

// The 84 vector instructions that dequantise a step (21 per packed word: code = word * 21 + u, u as in
// dequant_op below) in the order and grouping in which they go between the MFMAs of the step before: 54
// units of one or two instructions, never split over two MFMAs.  A packed-fp16 instruction right before an
// MFMA costs a wait state, so each of them (the subtractions u = 9..12 and multiplications 13..16) is
// followed by an instruction of the next word that does not depend on it (its constants 0..3, shift 4 and
// extractions 5..8; words alternate between two sets of temporaries); the re-ordering (17..20) of word 2 is
// held back to pair with the subtractions of word 3, whose first two multiplications stay alone.
constexpr int kTallUnits = 54;
constexpr signed char kTallSchedule[kTallUnits][2] = {
    {0, -1}, {1, -1}, {2, -1}, {3, -1}, {4, -1}, {5, -1}, {6, -1}, {7, -1}, {8, -1},
    {9, 21}, {10, 22}, {11, 23}, {12, 24}, {13, 25}, {14, 26}, {15, 27}, {16, 28}, {29, -1},
    {17, -1}, {18, -1}, {19, -1}, {20, -1}, {30, 42}, {31, 43}, {32, 44}, {33, 45}, {34, 46},
    {35, 47}, {36, 48}, {37, 49}, {50, -1}, {38, -1}, {39, -1}, {40, -1}, {41, -1}, {51, 63},
    {52, 64}, {53, 65}, {54, 66}, {55, 67}, {56, 68}, {57, 69}, {58, 70}, {71, -1}, {72, 59},
    {73, 60}, {74, 61}, {75, 62}, {76, -1}, {77, -1}, {78, 80}, {79, 81}, {82, -1}, {83, -1},
};

// The A operands are read from LDS by hand as well: the compiler waits before the first use of every one
// of them (sixteen waits per round at sixteen row tiles), four tiles at a time are enough.
template <int OFFSET>
__device__ __forceinline__ void tall_lds_read(half8_t& dst, uint32_t addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFFSET) : "memory");
}
// Everything but the newest NEWEST LDS reads has arrived; the operands read next pass through the wait.
template <int NEWEST, int COUNT>
__device__ __forceinline__ void tall_lds_wait(half8_t* a) {
    if constexpr (COUNT == 4)
        asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]) : "n"(NEWEST) : "memory");
    else
        asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a[0]), "+v"(a[1]) : "n"(NEWEST) : "memory");
}

// MT: 16-row MFMA tiles per block of rows (8: blocks of 128 rows; 4: one block of up to 64 rows; 2: up to 32
// rows, reached only when MH_GEMM_TALL_MIN_M is lowered), the same walk with fewer MFMAs per dequantised word.
// NS: rounds in flight = slots of the register ring = activation stages in LDS.  Four everywhere: eight (the
// LDS allows them below eight row tiles) measured slower, 32 x 8192 x 57344 90.3 against 77.8 us and 64 x 8192 x
// 10240 30.3 against 29.0 -- what holds the kernel back at few rows is its ~105 vector instructions per
// round, not latency.
template <int MT, int NS>
__global__ __launch_bounds__(tall_k_shares(MT) * 128) void gptq_gemm_tall_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ qweight, const uint32_t* __restrict__ qzeros,
    const half_t* __restrict__ scales, half_t* __restrict__ out, float* __restrict__ partial, int M, int N, int K,
    int group_size, int rounds_per_block, int split_k, const half_t* __restrict__ bias, int epilogue) {
    constexpr int BM = 16 * MT;
    constexpr int KS = tall_k_shares(MT);          // waves per column group, each with 32 k of every round
    constexpr int RK = 32 * KS;                    // k per round
    constexpr int kThreads = 2 * KS * 64;
    constexpr int kHalfBytes = BM * 128;           // [row][64 k], chunks swizzled
    constexpr int kStageBytes = (RK / 64) * kHalfBytes;  // the halves of a round's k
    constexpr int PW = MT / 2;                     // 1 KiB pieces of a stage per wave
    constexpr int LR = 3 + PW;                     // loads per wave and round
    constexpr int kRegion = MT * 4096;             // a wave's accumulators in LDS
    static_assert(MT == 2 || MT == 4 || MT == 8 || MT == 16, "two, four, eight or sixteen row tiles");
    __shared__ __attribute__((aligned(1024))) int8_t smem[NS * kStageBytes];
    static_assert(NS * kStageBytes >= KS * kRegion, "the reduction reuses the stages");

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int cg = wave & 1, ks = wave >> 1;
    const int j = lane & 15, o = lane >> 4;
    const int n0 = blockIdx.x * kTallBN, m0 = blockIdx.z * BM;
    const int rounds_total = K / RK;
    const int r_begin = blockIdx.y * rounds_per_block;
    const int n_rounds = min(rounds_per_block, rounds_total - r_begin);
    // this wave's 32 k of the workgroup's first round
    const int k_wave = r_begin * RK + ks * 32;
    // first of the lane's four columns.  kEpilogueSiluPairs (columns in blocks of 128 gate + 128 up): the
    // tile is 64 gate columns (cg = 0) and the 64 matching up columns (cg = 1) of block blockIdx.x / 2
    const bool silu = epilogue == kEpilogueSiluPairs;
    const int pair_col = (blockIdx.x >> 1) * 256 + cg * 128 + (blockIdx.x & 1) * 64;
    const int col = (silu ? pair_col : n0 + cg * 64) + 4 * j;

    // the descriptors live in fixed scalar registers; past the workgroup's last round their record count is
    // set to zero (one scalar instruction), and a load moves nothing and returns zeros
    int4_t x_rsrc = tall_rsrc(x, (uint32_t)((size_t)M * K * 2));
    int4_t w_rsrc = tall_rsrc(qweight, (uint32_t)((size_t)(K / 8) * N * 4));
    int4_t s_rsrc = tall_rsrc(scales, (uint32_t)((size_t)(K / group_size) * N * 2));
    int4_t z_rsrc = tall_rsrc(qzeros, (uint32_t)((size_t)(K / group_size) * (N / 8) * 4));
    const int x_bytes = x_rsrc[2], w_bytes = w_rsrc[2], s_bytes = s_rsrc[2], z_bytes = z_rsrc[2];

    // ---- what a lane fetches per round
    // activations: of the stage's 4 MT pieces of 1 KiB (half h, rows 8p .. 8p+7) this wave loads h = wave / 4,
    // p = (wave % 4) * PW + i; lane l lands at row 8p + l / 8, chunk position l % 8, which holds the
    // chunk (l % 8) ^ swizzle(row); rows past M are past the end of the buffer and read as zero
    int x_off[PW];
#pragma unroll
    for (int i = 0; i < PW; ++i) {
        const int row = ((wave & 3) * PW + i) * 8 + (lane >> 3);
        const int chunk = (lane & 7) ^ ((row >> 1) & 7);
        x_off[i] = ((m0 + row) * K + r_begin * RK + (wave >> 2) * 64 + chunk * 8) * 2;
        // the odd pieces ride on the even ones' write of m0 with an instruction offset of 1 KiB
        // (row >= 8 there and K >= 512: the offset stays positive)
        if (PW > 1 && (i & 1)) x_off[i] -= 1024;
    }
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(size_t)smem);
    const uint32_t lds_wave = lds0 + (uint32_t)(wave >> 2) * kHalfBytes + (uint32_t)((wave & 3) * PW) * 1024u;
    const int w_off = ((k_wave / 8 + o) * N + col) * 4;
    const int s_off = col * 2, z_off = (col >> 3) * 4;
    const int z_shift = (j & 1) * 16;  // the lane's four zero points: nibbles 4 (j & 1) .. + 3 of the word

    uint4_t rq[NS];   // packed words of steps r .. r + NS - 1
    uint2_t rs[NS];   // their scales
    uint32_t rz[NS];  // their zero-point words
    // group of the step whose loads are issued next / whose constants are built next
    int load_group = __builtin_amdgcn_readfirstlane(k_wave / group_size);
    int load_in_group = __builtin_amdgcn_readfirstlane(k_wave % group_size);
    // The LR loads that go with step `step`, in their fixed order: piece 0 the packed words, 1 the scales,
    // 2 the zero points (all into ring slot S), 3.. the wave's 1 KiB pieces of the activation stage of round
    // step - 1 (into buffer (step - 1) % NS).  The main loop spreads the pieces over the round's MFMAs: issued
    // back to back by all eight waves right after the barrier they fill the vector memory queue, and the
    // waves stall in issue with the matrix pipes idle.
    auto issue_piece = [&](auto slot, auto piece, int step) {
        constexpr int S = decltype(slot)::value, I = decltype(piece)::value;
        const bool live = step < n_rounds;
        if constexpr (I == 0) {
            w_rsrc[2] = live ? w_bytes : 0;
            tall_load_b128_stream(rq[S], w_off, w_rsrc, step * (RK / 2) * N);
        }
        if constexpr (I == 1) {
            s_rsrc[2] = live ? s_bytes : 0;
            tall_load_b64(rs[S], s_off, s_rsrc, __builtin_amdgcn_readfirstlane(load_group * N * 2));
        }
        if constexpr (I == 2) {
            z_rsrc[2] = live ? z_bytes : 0;
            tall_load_b32(rz[S], z_off, z_rsrc, __builtin_amdgcn_readfirstlane(load_group * (N / 8) * 4));
            load_in_group += RK;
            while (load_in_group >= group_size) {
                load_in_group -= group_size;
                ++load_group;
            }
        }
        if constexpr (I >= 3) {
            const int stage = step - 1;
            const uint32_t base = lds_wave + (uint32_t)((S + NS - 1) % NS) * kStageBytes;
            if constexpr (I == 3) x_rsrc[2] = stage < n_rounds ? x_bytes : 0;
            if constexpr (PW == 1)
                tall_load_to_lds(base, x_off[0], x_rsrc, stage * (RK * 2));
            else if constexpr ((I - 3) % 2 == 0)
                tall_load_to_lds_pair(base + (uint32_t)(I - 3) * 1024u, x_off[I - 3], x_off[I - 2], x_rsrc, stage * (RK * 2));
        }
    };
    auto issue = [&](auto slot, int step, bool with_stage) {
        issue_piece(slot, std::integral_constant<int, 0>{}, step);
        issue_piece(slot, std::integral_constant<int, 1>{}, step);
        issue_piece(slot, std::integral_constant<int, 2>{}, step);
        if (with_stage) tall_static_for<3, LR>([&](auto piece) { issue_piece(slot, piece, step); });
    };

    DequantRegs regs;
    regs.init(4);
    ColumnConst cc[4];
    // The constants of make_column_const() without conversions, four instructions per column: for a zero
    // point z <= 15 the fp16 values 1024 + (z + 1) and 64 + (z + 1) are 0x6400 + (z + 1) and 0x5400 +
    // 16 (z + 1) as bit patterns (one unit, one sixteenth per mantissa step), so both pairs are one
    // 24-bit multiply-add of z each.
    auto make_const = [&](int c, const uint2_t& s, uint32_t z) {
        const uint32_t zc = (z >> (z_shift + 4 * c)) & 0xFu;
        const uint32_t sw = s[c >> 1];
        cc[c].scale = as_half2((c & 1) ? __builtin_amdgcn_perm(sw, sw, 0x07060706u) : __builtin_amdgcn_perm(sw, sw, 0x05040504u));
        cc[c].zero_lo = as_half2(zc * 0x00010001u + 0x64016401u);
        cc[c].zero_hi = as_half2(zc * 0x00100010u + 0x54105410u);
    };
    auto make_consts = [&](const uint2_t& s, uint32_t z) {
#pragma unroll
        for (int c = 0; c < 4; ++c) make_const(c, s, z);
    };
    // one packed word -> the B operand of MFMA tile c: k0 .. k7 of column 4j + c
    auto dequant_piece = [&](half8_t& b, uint32_t word, int c) {
        half2_t w[4];
        dequant_word<4>(word, cc[c], regs, w);
        b = half8_t{w[0][0], w[1][0], w[2][0], w[3][0], w[0][1], w[1][1], w[2][1], w[3][1]};
    };
    // The same arithmetic (dequant_word<4>, the constants above) one instruction at a time, 21 per packed
    // word: a wave issues one instruction of any kind in about five cycles, so whatever stands between two
    // of its MFMAs beyond two or three instructions leaves the matrix pipe waiting.  Instruction u of word c
    // reads packed word `word` and the step's scales and zero points; the last four write the B operand
    // registers.  Dependent instructions are at least three apart (next to each other they cost a wait
    // state); the empty statement pins each between the MFMAs it was written between: pure arithmetic is
    // otherwise placed next to its use, a round later, in one block.
    ColumnConst kc[2];
    uint32_t zc[2], q8[2];
    half2_t wq[2][4];
    auto dequant_op = [&](auto op_c, uint4_t& bw, const uint4_t& q4, int c, const uint2_t& sc, uint32_t z) {
        constexpr int u = decltype(op_c)::value % 21, e = (decltype(op_c)::value / 21) & 1;
        const half2_t sixteenth = half2_t{(half_t)0.0625f, (half_t)0.0625f};
        const uint32_t sw = sc[c >> 1], word = q4[c];
        auto pin = [&](auto& out) { asm volatile("" : "+v"(out)); };
        if constexpr (u == 0) { zc[e] = (z >> (z_shift + 4 * c)) & 0xFu; pin(zc[e]); }
        if constexpr (u == 1) {
            kc[e].scale = as_half2((c & 1) ? __builtin_amdgcn_perm(sw, sw, 0x07060706u) : __builtin_amdgcn_perm(sw, sw, 0x05040504u));
            pin(kc[e].scale);
        }
        if constexpr (u == 2) { kc[e].zero_lo = as_half2(__umul24(zc[e], 0x00010001u) + 0x64016401u); pin(kc[e].zero_lo); }
        if constexpr (u == 3) { kc[e].zero_hi = as_half2(__umul24(zc[e], 0x00100010u) + 0x54105410u); pin(kc[e].zero_hi); }
        if constexpr (u == 4) { q8[e] = word >> 8; pin(q8[e]); }
        if constexpr (u >= 5 && u <= 8) {
            constexpr int i = u - 5;
            wq[e][i] = as_half2(((i < 2 ? word : q8[e]) & ((i & 1) ? regs.mask_hi : regs.mask_lo)) | regs.magic);
            pin(wq[e][i]);
        }
        if constexpr (u >= 9 && u <= 12) {
            constexpr int i = u - 9;
            wq[e][i] = (i & 1) ? __builtin_elementwise_fma(wq[e][i], sixteenth, -kc[e].zero_hi) : wq[e][i] - kc[e].zero_lo;
            pin(wq[e][i]);
        }
        if constexpr (u >= 13 && u <= 16) {
            wq[e][u - 13] = wq[e][u - 13] * kc[e].scale;
            pin(wq[e][u - 13]);
        }
        if constexpr (u >= 17) {
            // registers of the operand: (k0 k1) (k2 k3) (k4 k5) (k6 k7) from the pairs (k0 k4) (k1 k5) (k2 k6) (k3 k7)
            constexpr int i = u - 17, pr = (i >> 1) * 2;
            uint32_t r = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, wq[e][pr + 1]), __builtin_bit_cast(uint32_t, wq[e][pr]),
                                               (i & 1) ? 0x07060302u : 0x05040100u);
            pin(r);
            bw[(i & 1) * 2 + (i >> 1)] = r;
        }
    };

    // A operand of row tile rt: row rt*16 + j, chunk (ks & 1)*4 + o of the wave's half; the swizzle of
    // row rt*16 + j does not depend on rt
    const int a_off = tall_swz(j, (ks & 1) * 4 + o);
    // Which row tile a wave keeps in accumulator rt differs between the waves that share a column group:
    // rt ^ own, own = the first of the row tiles that the wave ends up with when the K shares are added
    // (below): with four shares wave ks = 0 the first quarter of the row tiles, 2 the second, 1 the third, 3
    // the fourth; with two shares a half each.  Every wave then keeps its lowest accumulators and gives away
    // the others, and no branch decides which registers are touched.  kOwn: row tiles per owner.  (Two row
    // tiles: wave 0 takes all, own = 0.)
    constexpr int kOwn = MT < 4 ? MT : (KS == 4 ? MT / 4 : MT / 2);
    const int own = MT < 4 ? 0 : KS == 4 ? (MT / 2) * (ks & 1) + (MT / 4) * (ks >> 1) : (MT / 2) * ks;
    // LDS offset of the first of the row tiles behind accumulators [g kOwn, (g + 1) kOwn)
    int a_group_off[MT / kOwn];
#pragma unroll
    for (int g = 0; g < MT / kOwn; ++g) a_group_off[g] = a_off + ((g * kOwn) ^ own) * 2048;
    float4_t acc[MT][4];
#pragma unroll
    for (int rt = 0; rt < MT; ++rt)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[rt][c] = float4_t{0.f, 0.f, 0.f, 0.f};
    uint4_t bw[2][4];  // B operands of two steps, as registers

    // ---- prologue: the loads of the virtual rounds -NS .. -1, then the operands of step 0
    tall_static_for<0, NS>([&](auto slot) { issue(slot, decltype(slot)::value, decltype(slot)::value != 0); });
    tall_wait<0>(rq[0], rs[0], rz[0]);
    make_consts(rs[0], rz[0]);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        half8_t b0;
        dequant_piece(b0, rq[0][c], c);
        bw[0][c] = __builtin_bit_cast(uint4_t, b0);
    }

    // ---- one round: S = r % NS (ring slot, stage buffer), P = r % 2 (B operand set; NS is even)
    static_assert(NS % 2 == 0, "the B operand sets alternate with the rounds");
    auto round = [&](auto slot, int r) {
        constexpr int S = decltype(slot)::value, P = S & 1, S1 = (S + 1) % NS;
        // done after this wait: everything up to the stage of round r, which includes the words and
        // constants of step r + 1; still in flight: the LR loads of each of the last NS - 2 rounds
        tall_wait<(NS - 2) * LR>(rq[S1], rs[S1], rz[S1]);
        __syncthreads();
        // from here on slot S is free (step r was dequantised last round) and so is the stage buffer of
        // round r - 1: the loads of step r + NS and stage r + NS - 1 go out between the MFMAs below
        half8_t a[MT];
        const uint32_t a_stage = lds0 + (uint32_t)(S * kStageBytes + (ks >> 1) * kHalfBytes);
        tall_static_for<0, MT>([&](auto rt) {
            tall_lds_read<(decltype(rt)::value % kOwn) * 2048>(a[decltype(rt)::value], a_stage + (uint32_t)a_group_off[decltype(rt)::value / kOwn]);
        });
        __builtin_amdgcn_sched_barrier(0);
        // 4 MT MFMAs; after MFMA m its share of the 54 units that dequantise step r + 1 and, after
        // every fourth (second at four row tiles, every one at two), one of the round's loads
        tall_static_for<0, 4 * MT>([&](auto mfma) {
            constexpr int m = decltype(mfma)::value;
            constexpr int G = MT < 4 ? MT : 4;  // row tiles per wait
            if constexpr (m % (4 * G) == 0) tall_lds_wait<MT - (m / 4 + G), G>(&a[m / 4]);
            acc[m >> 2][m & 3] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[m >> 2], __builtin_bit_cast(half8_t, bw[P][m & 3]),
                                                                        acc[m >> 2][m & 3], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            constexpr int load = MT >= 8 ? (m % 4 == 3 ? m / 4 : -1) : MT == 4 ? (m % 2 == 1 ? m / 2 : -1) : m;
            if constexpr (load >= 0 && load < LR) issue_piece(slot, std::integral_constant<int, load>{}, r + NS);
            tall_static_for<m * kTallUnits / (4 * MT), (m + 1) * kTallUnits / (4 * MT)>([&](auto unit) {
                constexpr int first = kTallSchedule[decltype(unit)::value][0], second = kTallSchedule[decltype(unit)::value][1];
                dequant_op(std::integral_constant<int, first>{}, bw[P ^ 1][first / 21], rq[S1], first / 21, rs[S1], rz[S1]);
                if constexpr (second >= 0)
                    dequant_op(std::integral_constant<int, second>{}, bw[P ^ 1][second / 21], rq[S1], second / 21, rs[S1], rz[S1]);
            });
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    for (int r = 0; r < n_rounds; r += NS)
        tall_static_for<0, NS>([&](auto slot) {
            if (r + decltype(slot)::value < n_rounds) round(slot, r + decltype(slot)::value);
        });

    // the loads requested past the end are still in flight: their registers are dead to the compiler
    // and their stages would land in LDS that the reduction is about to use
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    // ---- the K shares of the waves, added in a fixed order: (0 + 1) + (2 + 3)
    // Waves ks and ks ^ 1 exchange halves of their accumulators, then (four shares) ks and ks ^ 2 halves of
    // what is left: every wave moves data at every step and ends up with kOwn row tiles, fully summed, in
    // its lowest accumulators (row tiles own .. own + kOwn - 1).  With one wave collecting everything, three
    // quarters of the waves sat idle for most of the 4 us behind the main loop.  a + b and b + a are the same
    // bits, so the sums are those of the tree above whichever wave forms them.
    // row tiles in accumulators [FIRST, FIRST + COUNT) as COUNT x 4 blocks of 1 KiB, lane-linear on both sides
    auto put_tiles = [&](auto first, auto count, int8_t* slot) {
        float4_t* dst = reinterpret_cast<float4_t*>(slot) + lane;
        tall_static_for<0, decltype(count)::value * 4>([&](auto i) {
            dst[decltype(i)::value * 64] = acc[decltype(first)::value + decltype(i)::value / 4][decltype(i)::value % 4];
        });
    };
    auto add_tiles = [&](auto first, auto count, const int8_t* slot) {
        const float4_t* src = reinterpret_cast<const float4_t*>(slot) + lane;
        tall_static_for<0, decltype(count)::value * 4>([&](auto i) {
            acc[decltype(first)::value + decltype(i)::value / 4][decltype(i)::value % 4] += src[decltype(i)::value * 64];
        });
    };
    if constexpr (MT >= 4) {
        constexpr int H = MT / 2;
        put_tiles(std::integral_constant<int, H>{}, std::integral_constant<int, H>{}, smem + wave * (H * 4096));
        __syncthreads();
        add_tiles(std::integral_constant<int, 0>{}, std::integral_constant<int, H>{}, smem + (wave ^ 2) * (H * 4096));
        __syncthreads();
        if constexpr (KS == 4) {
            constexpr int Q = MT / 4;
            put_tiles(std::integral_constant<int, Q>{}, std::integral_constant<int, Q>{}, smem + wave * (Q * 4096));
            __syncthreads();
            add_tiles(std::integral_constant<int, 0>{}, std::integral_constant<int, Q>{}, smem + (wave ^ 4) * (Q * 4096));
            __syncthreads();
        }
    } else {
        // two row tiles: a wave's accumulators as 4 MT blocks of 1 KiB; wave ks = 0 collects
        auto put = [&](int region) { put_tiles(std::integral_constant<int, 0>{}, std::integral_constant<int, MT>{}, smem + region * kRegion); };
        auto add = [&](int region) { add_tiles(std::integral_constant<int, 0>{}, std::integral_constant<int, MT>{}, smem + region * kRegion); };
        if (ks & 1) put((ks >> 1) * 2 + cg);
        __syncthreads();
        if (!(ks & 1)) add((ks >> 1) * 2 + cg);
        __syncthreads();
        if (ks == 2) put(cg);
        __syncthreads();
        if (ks == 0) add(cg);
        __syncthreads();
    }
    const bool owner = MT >= 4 || ks == 0;  // holds sums to store

    // ---- results: acc[rt][c][e], rt < kOwn, is row (own + rt)*16 + o*4 + e, column cg*64 + 4j + c of the tile
    if (split_k == 1) {
        constexpr int kRow = 256 + 16;  // bytes per tile row in LDS
        if (owner) {
#pragma unroll
            for (int rt = 0; rt < kOwn; ++rt)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const half4_t h = {(half_t)acc[rt][0][e], (half_t)acc[rt][1][e], (half_t)acc[rt][2][e], (half_t)acc[rt][3][e]};
                    *reinterpret_cast<half4_t*>(smem + ((own + rt) * 16 + o * 4 + e) * kRow + (cg * 64 + 4 * j) * 2) = h;
                }
        }
        __syncthreads();
        if (silu) {
            // out[m, b*128 + h*64 + c] = silu(gate) * up of the fp16-rounded sums, b = blockIdx.x / 2, h = blockIdx.x % 2
            half_t* dst = out + (blockIdx.x >> 1) * 128 + (blockIdx.x & 1) * 64;
#pragma unroll
            for (int i = 0; i < (BM * 8 + kThreads - 1) / kThreads; ++i) {
                const int id = i * kThreads + tid, row = id >> 3, ch = id & 7;
                if (row >= BM || m0 + row >= M) continue;
                const half8_t g = *reinterpret_cast<const half8_t*>(smem + row * kRow + ch * 16);
                const half8_t u = *reinterpret_cast<const half8_t*>(smem + row * kRow + 128 + ch * 16);
                half8_t h;
#pragma unroll
                for (int e = 0; e < 8; ++e) h[e] = silu_pair(g[e], u[e]);
                *reinterpret_cast<half8_t*>(dst + (size_t)(m0 + row) * (N / 2) + ch * 8) = h;
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < BM * 16 / kThreads; ++i) {
            const int id = i * kThreads + tid, row = id >> 4, ch = id & 15;
            const int m = m0 + row, n = n0 + ch * 8;
            if (m >= M || n >= N) continue;
            half8_t h = *reinterpret_cast<const half8_t*>(smem + row * kRow + ch * 16);
            if (bias) h = h + *reinterpret_cast<const half8_t*>(bias + n);
            *reinterpret_cast<half8_t*>(out + (size_t)m * N + n) = h;
        }
    } else if constexpr (MT <= 8) {  // (sixteen row tiles: the fp32 tile does not fit the LDS; the plan never splits K there)
        constexpr int kRow = 512 + 16;
        if (owner) {
#pragma unroll
            for (int rt = 0; rt < kOwn; ++rt)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float4_t v = {acc[rt][0][e], acc[rt][1][e], acc[rt][2][e], acc[rt][3][e]};
                    *reinterpret_cast<float4_t*>(smem + ((own + rt) * 16 + o * 4 + e) * kRow + (cg * 64 + 4 * j) * 4) = v;
                }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < BM * 32 / kThreads; ++i) {
            const int id = i * kThreads + tid, row = id >> 5, ch = id & 31;
            const int m = m0 + row, n = n0 + ch * 4;
            if (m >= M || n >= N) continue;
            *reinterpret_cast<float4_t*>(partial + ((size_t)blockIdx.y * M + m) * N + n) =
                *reinterpret_cast<const float4_t*>(smem + row * kRow + ch * 16);
        }
    }
}

// ---- host side ---------------------------------------------------------------------------

struct TallPlan {
    int mt, tiles_n, row_blocks, split_k, rounds_per_block;
};

// MH_GEMM_TALL_MT16: 0 never blocks of 256 rows, 1 (default) where they pad the rows no further than blocks
// of 128 and fill the CUs without a split of K, 2 wherever K need not be split.
static int tall_mt16_mode() {
    static const int v = [] {
        const char* e = getenv("MH_GEMM_TALL_MT16");
        return e && *e ? atoi(e) : 1;
    }();
    return v;
}

static TallPlan plan_tall(int M, int N, int K) {
    TallPlan p;
    p.mt = M <= 32 ? 2 : M <= 64 ? 4 : 8;
    p.tiles_n = (N + kTallBN - 1) / kTallBN;
    if (M > 128 && tall_mt16_mode() != 0) {
        // blocks of 256 rows: one wave per SIMD, a packed word dequantised once per 256 rows; the whole K per
        // workgroup (its fp32 tile would not fit the LDS for a split)
        const int blocks = (M + 255) / 256;
        const bool same_padding = blocks * 256 == (M + 127) / 128 * 128;
        if ((same_padding || tall_mt16_mode() == 2) && (long)p.tiles_n * blocks * 8 >= (long)compute_units() * 7) {
            p.mt = 16;
            p.row_blocks = blocks;
            p.split_k = 1;
            p.rounds_per_block = K / (32 * tall_k_shares(16));
            return p;
        }
    }
    const int bm = 16 * p.mt;
    p.row_blocks = (M + bm - 1) / bm;
    const int rounds = K / kTallRoundK;
    // one workgroup per CU (eight waves; 128 KiB of LDS at eight row tiles); a workgroup keeps at least four
    // rounds, and the fp32 partial sums (8 M N bytes per split, written and read) stay below the packed
    // weights' bytes -- or below twice those where that shortens a workgroup's walk by a quarter or more
    // (4096 x 4096 at 128 rows 23.0 us with two K ranges against 19.8 with four, 5120 x 5120 26.9 / 22.9,
    // 1024 x 8192 21.5 / 16.9; below four times: 21.4, 23.8, 16.8; 4096 x 14336 at 128 rows measures the
    // same with seven and with eight ranges and keeps seven)
    long most = (long)compute_units() / ((long)p.tiles_n * p.row_blocks);
    if (most > rounds / 4) most = rounds / 4;
    const long rows = M < bm ? M : bm;
    auto capped = [&](long per_rows) {
        long split = (long)K / (per_rows * rows);
        if (split > most) split = most;
        return split < 1 ? 1L : split;
    };
    long split = capped(16);
    const long relaxed = capped(8);
    if (((rounds + relaxed - 1) / relaxed) * 4 <= ((rounds + split - 1) / split) * 3) split = relaxed;
    p.rounds_per_block = (int)((rounds + split - 1) / split);
    p.split_k = (rounds + p.rounds_per_block - 1) / p.rounds_per_block;
    return p;
}

// MH_GEMM_TALL_MIN_M: the fewest rows that come here whatever the shape (default 33); 0: unset.
static int tall_min_m_env() {
    static const int v = [] {
        const char* e = getenv("MH_GEMM_TALL_MIN_M");
        return e && *e ? atoi(e) : 0;
    }();
    return v;
}

// 17 to 32 rows (two row tiles): this kernel where its workgroups are many and their walks short, i.e. where
// a launch is made of fixed costs rather than of its weight stream.  Measured at 24 rows against the
// small-M kernel (us, this kernel / small-M): 13824 x 5120 (240 workgroups, 18 rounds) 16.9 / 24.4, 4096 x
// 12288 (192, 16) 15.6 / 20.1, 4096 x 28672 (224, 32) 20.1 / 23.8, 17920 x 6656 (208, 35) 24.7 / 26.0, 8192 x
// 16384 (256, 32) 24.1 / 25.2, 8192 x 8192 16.5 / 17.5, 4096 x 4096 10.0 / 10.7; but 8192 x 28672 (224
// workgroups, 64 rounds) 36.5 / 36.2, 28672 x 8192 (256, 56) 37.0 / 34.6, 8192 x 22016 (172, 64) 36.0 / 32.5,
// 6656 x 17920 (140 workgroups) 29.5 / 25.4.  Up to 16 rows the small-M kernel's single row tile wins
// nearly everywhere (8192 x 8192 12.3 against 15.7).
static bool tall_two_row_tiles_preferred(int M, int N, int K) {
    if (M < 17 || M > 32) return false;
    const TallPlan p = plan_tall(M, N, K);
    return (long)p.tiles_n * p.split_k * 8 >= (long)compute_units() * 5 && p.rounds_per_block <= 40;
}

// Measured on one box against what served these shapes before (the small-M kernel's 64-row blocks up to
// 191 rows, the LDS-staged kernel above; us, this kernel / before): 4096 x 28672 at 65 / 128 / 256 / 2048
// rows 38.7 / 58.6, 41.2 / 62.3, 75.2 / 80.5, 561 / 567; 4096 x 14336: 29.1 / 33.0, 36.5 / 35.9, 40.1 /
// 55.3, 278 / 310; 14336 x 4096: 28.3 / 33.8, 32.2 / 33.1, 43.1 / 60.0, 242 / 283; 8192 x 8192 at 512 rows
// 72.0 / 113.5.  Never slower by more than 2 %, so every 4-bit product of more than 64 rows whose K is a
// multiple of 128 comes here.  With four row tiles (33 to 64 rows) against the small-M kernel's single block
// of 64 rows, at 64 rows: 8192 x 10240 29.0 / 41.6, 28672 x 8192 55.7 / 62.3, 4096 x 14336 23.9 / 26.3, 8192 x
// 57344 109 / 112; with two row tiles at 32 rows it loses on the largest shapes (8192 x 57344 77.8 / 67.9, 28672
// x 8192 48.6 / 43.5: there the weight stream dominates and the small-M kernel's ring of eight loads per
// wave hides more latency than this kernel's three rounds), so every shape comes here from 33 rows and
// the shapes of tall_two_row_tiles_preferred from 17 (MH_GEMM_TALL_MIN_M sets one switch for all).
// (These figures predate the dequantisation in parts, which made every shape 2-6 % faster.)  A round of 128 k
// needs 1,765 cycles whatever the data against the 1,024 of its MFMAs (instruction issue: two vector
// instructions per MFMA are free, the loop has 2.6 plus its scalar ones), and random operands cost 13-19 %
// of the clock on top (power).
bool gemm_tall_preferred(int M, int N, int K, int group_size, int bits, int epilogue) {
    static const char* off = getenv("MH_GEMM_NO_TALL");
    if (off && *off && atoi(off)) return false;
    if (!(bits == 4 && epilogue == kEpilogueNone && K % kTallRoundK == 0 && K >= 4 * kTallRoundK &&
          group_size % 32 == 0 && K % group_size == 0 && N % 8 == 0 && (size_t)M * K * 2 < ((size_t)1 << 31) &&
          (size_t)K * N / 2 < ((size_t)1 << 31)))
        return false;
    if (tall_min_m_env() > 0) return M >= tall_min_m_env();
    return M >= 33 || tall_two_row_tiles_preferred(M, N, K);
}

size_t gemm_tall_workspace_bytes(int M, int N, int K) {
    const TallPlan p = plan_tall(M, N, K);
    return p.split_k > 1 ? kTileCounterBytes + (size_t)p.split_k * M * N * sizeof(float) : 0;
}

// kEpilogueSiluPairs in the kernel's own store: an unsplit plan, whole blocks of 128 + 128 columns.
bool gemm_tall_silu_pairs_supported(int M, int N, int K, int group_size, int bits) {
    return gemm_tall_preferred(M, N, K, group_size, bits, kEpilogueNone) && N % 256 == 0 && plan_tall(M, N, K).split_k == 1;
}

int gptq_gemm_tall_launch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                          const void* scales, void* out, int M, int N, int K, int group_size, void* workspace,
                          size_t workspace_bytes, const half_t* bias, int epilogue) {
    const TallPlan p = plan_tall(M, N, K);
    if (epilogue != kEpilogueNone && (epilogue != kEpilogueSiluPairs || p.split_k != 1 || N % 256 != 0 || bias))
        return fail(MH_ERR_INVALID, "gptq gemm (128-row blocks): epilogue %d is not served for M=%d N=%d K=%d", epilogue, M, N, K);
    const size_t need = gemm_tall_workspace_bytes(M, N, K);
    if (need != 0 && (workspace == nullptr || workspace_bytes < need))
        return fail(MH_ERR_WORKSPACE, "mh_gptq_gemm: workspace of %zu bytes required, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    float* partial = need ? reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + kTileCounterBytes) : nullptr;
#define MH_LAUNCH_TALL(MT)                                                                                            \
    hipLaunchKernelGGL((gptq_gemm_tall_kernel<MT, 4>), dim3(p.tiles_n, p.split_k, p.row_blocks),                     \
                       dim3(tall_k_shares(MT) * 128), 0,                                                              \
                       stream, (const half_t*)x, (const uint32_t*)qweight, (const uint32_t*)qzeros,                  \
                       (const half_t*)scales, (half_t*)out, partial, M, N, K, group_size, p.rounds_per_block,        \
                       p.split_k, bias, epilogue)
    switch (p.mt) {
        case 2: MH_LAUNCH_TALL(2); break;
        case 4: MH_LAUNCH_TALL(4); break;
        case 16: MH_LAUNCH_TALL(16); break;
        default: MH_LAUNCH_TALL(8); break;
    }
#undef MH_LAUNCH_TALL
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
