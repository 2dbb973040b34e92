// GPTQ w4a16 / w8a16 dequant-GEMM on CDNA4 fp16 MFMA (v_mfma_f32_16x16x32_f16).
//
// Replaces the fused qmm kernel of the reference
// (examples/qwen1_5_int8.py:156-216) for M above the GEMV range.
//
// Mapping.  The B operand of a 16x16x32 MFMA wants, in lane l, eight
// consecutive k of column l % 16, k-chunk l / 16 -- for 4-bit GPTQ that is
// exactly one packed word of qweight.  A lane therefore loads 16 bytes (four
// adjacent columns of one packed row), dequantises each word in registers
// (gptq_common.h) and feeds it to one of four MFMAs; the weights never touch
// LDS.  The order of k inside a word that the extraction produces is applied to
// the activations instead, when they are staged into LDS, so both operands
// agree.  A block is four waves side by side along N (256 columns, 1 KiB
// contiguous per packed row) sharing one activation tile [16*MT, KC] in LDS.
// K is split over blockIdx.y with fp32 partials summed in split order by a
// second, tiny kernel (deterministic; see gptq_gemv.hip).
#include "gptq_common.h"

namespace mh {

#pragma clang fp contract(off)

constexpr int kGemmCols = 256;
constexpr int kGemmDepth = 4;  // weight prefetch distance in k-steps

template <int MT> struct GemmStage { static constexpr int kSteps = MT <= 2 ? 16 : (MT == 4 ? 8 : 4); };

template <int BITS, int MT>
__global__ __launch_bounds__(256) void gptq_gemm_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ qweight,
    const uint32_t* __restrict__ qzeros, const half_t* __restrict__ scales,
    half_t* __restrict__ out, float* __restrict__ partial,
    int M, int N, int K, int steps_per_group, int steps_total, int steps_per_block, int split_k) {
    constexpr int P = Packing<BITS>::kPerWord;
    constexpr int PAIRS = Packing<BITS>::kPairs;
    constexpr uint32_t MASK = Packing<BITS>::kMask;
    constexpr int BM = 16 * MT;
    constexpr int ROWS_PER_STEP = 32 / P;     // packed rows per 32-k step
    constexpr int LOADS = ROWS_PER_STEP / 4;  // 16-byte loads per lane per step
    constexpr int SC = GemmStage<MT>::kSteps; // k-steps per LDS stage
    constexpr int CHUNKS = SC * 4;            // 16-byte chunks per activation row per stage
    constexpr int RS = CHUNKS + 1;            // padded row stride in chunks
    constexpr int XLOADS = BM * CHUNKS / 256; // chunks each thread stages
    constexpr int D = kGemmDepth;
    static_assert(SC % D == 0, "stage must be a multiple of the prefetch depth");

    __shared__ uint4 xs[BM * RS];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nl = lane & 15, kq = lane >> 4;
    const int tile = blockIdx.x, split = blockIdx.y, mblock = blockIdx.z;
    const int m0 = mblock * BM;
    const int col = tile * kGemmCols + wave * 64 + nl * 4;
    const bool active = col < N;
    const int colc = active ? col : 0;

    const int step_begin = split * steps_per_block;
    const int step_end = min(steps_total, step_begin + steps_per_block);
    const int last_step = step_end - 1;

    DequantRegs regs;
    regs.init(BITS);

    float4_t acc[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[mt][t] = float4_t{0.f, 0.f, 0.f, 0.f};

    // ---- weight stream: ring of D steps in flight --------------------------------------
    uint4_t qb[D][LOADS];
    auto load_q = [&](int step, uint4_t* dst) {
        const int s = min(step, last_step);
        const size_t row = (size_t)s * ROWS_PER_STEP + kq * LOADS;
#pragma unroll
        for (int j = 0; j < LOADS; ++j)
            dst[j] = __builtin_nontemporal_load(
                reinterpret_cast<const uint4_t*>(qweight + (row + j) * N + colc));
    };
#pragma unroll
    for (int d = 0; d < D; ++d) load_q(step_begin + d, qb[d]);

    // ---- per-group constants, fetched one group ahead ------------------------------------
    uint2 s_next;
    uint32_t z_next;
    auto load_consts = [&](int g) {
        s_next = *reinterpret_cast<const uint2*>(scales + (size_t)g * N + colc);
        z_next = qzeros[(size_t)g * (N / P) + colc / P];
    };
    const int g_last = last_step / steps_per_group;
    int g_cur = step_begin / steps_per_group;
    load_consts(g_cur);
    ColumnConst cc[4];
    auto take_consts = [&]() {
        const uint32_t zword = z_next >> ((colc % P) * BITS);
        const half2_t s01 = as_half2(s_next.x), s23 = as_half2(s_next.y);
        cc[0] = make_column_const(s01.x, zword & MASK);
        cc[1] = make_column_const(s01.y, (zword >> BITS) & MASK);
        cc[2] = make_column_const(s23.x, (zword >> (2 * BITS)) & MASK);
        cc[3] = make_column_const(s23.y, (zword >> (3 * BITS)) & MASK);
    };
    take_consts();
    load_consts(min(g_cur + 1, g_last));

    // ---- activation staging -----------------------------------------------------------------
    uint4 xr[XLOADS];
    auto load_x = [&](int stage_step) {
#pragma unroll
        for (int it = 0; it < XLOADS; ++it) {
            const int idx = it * 256 + tid;
            const int row = idx / CHUNKS, chunk = idx % CHUNKS;
            const int m = m0 + row;
            const int step = stage_step + chunk / 4;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (m < M && step < step_end)
                v = *reinterpret_cast<const uint4*>(x + (size_t)m * K + (size_t)stage_step * 32 + chunk * 8);
            xr[it] = v;
        }
    };
    auto store_x = [&]() {
#pragma unroll
        for (int it = 0; it < XLOADS; ++it) {
            const int idx = it * 256 + tid;
            const int row = idx / CHUNKS, chunk = idx % CHUNKS;
            const uint32_t in[4] = {xr[it].x, xr[it].y, xr[it].z, xr[it].w};
            uint32_t o[4];
            if constexpr (BITS == 4) {
                pair_activations<4>(in, o);
            } else {
                pair_activations<8>(in, o);
                pair_activations<8>(in + 2, o + 2);
            }
            xs[row * RS + chunk] = make_uint4(o[0], o[1], o[2], o[3]);
        }
    };

    load_x(step_begin);
    for (int s0 = step_begin; s0 < step_end; s0 += SC) {
        __syncthreads();  // the previous stage has been consumed
        store_x();
        __syncthreads();
        if (s0 + SC < step_end) load_x(s0 + SC);

#pragma unroll
        for (int i = 0; i < SC; ++i) {
            const int step = s0 + i;
            const int g = min(step, last_step) / steps_per_group;
            if (g != g_cur) {
                g_cur = g;
                take_consts();
                load_consts(min(g + 1, g_last));
            }
            // B fragments: four columns, eight k each
            half8_t b[4];
            {
                uint4_t* q = qb[i % D];
                const uint32_t qa[4] = {q[0].x, q[0].y, q[0].z, q[0].w};
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    half2_t w[4];
                    if constexpr (BITS == 4) {
                        dequant_word<BITS>(qa[t], cc[t], regs, w);
                    } else {
                        const uint32_t qc[4] = {q[LOADS - 1].x, q[LOADS - 1].y, q[LOADS - 1].z, q[LOADS - 1].w};
                        dequant_word<BITS>(qa[t], cc[t], regs, w);
                        dequant_word<BITS>(qc[t], cc[t], regs, w + PAIRS);
                    }
                    const uint4_t packed = {as_u32(w[0]), as_u32(w[1]), as_u32(w[2]), as_u32(w[3])};
                    b[t] = __builtin_bit_cast(half8_t, packed);
                }
                load_q(step + D, q);
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const uint4 av = xs[(mt * 16 + nl) * RS + i * 4 + kq];
                const half8_t a = __builtin_bit_cast(half8_t, av);
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b[t], acc[mt][t], 0, 0, 0);
            }
        }
    }

    // ---- epilogue --------------------------------------------------------------------------------
    // acc[mt][t][r] is row m0 + mt*16 + kq*4 + r, column col + t.
    if (split_k == 1) {
        if (active) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int m = m0 + mt * 16 + kq * 4 + r;
                    if (m < M) {
                        const half4_t h = {(half_t)acc[mt][0][r], (half_t)acc[mt][1][r],
                                           (half_t)acc[mt][2][r], (half_t)acc[mt][3][r]};
                        *reinterpret_cast<half4_t*>(out + (size_t)m * N + col) = h;
                    }
                }
        }
        return;
    }

    // split-K: fp32 partials, summed in split order by splitk_finalize_kernel
    if (active) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + mt * 16 + kq * 4 + r;
                if (m < M) {
                    float* p = partial + ((size_t)split * M + m) * N + col;
                    *reinterpret_cast<float4_t*>(p) =
                        float4_t{acc[mt][0][r], acc[mt][1][r], acc[mt][2][r], acc[mt][3][r]};
                }
            }
    }
}

void launch_splitk_finalize(hipStream_t stream, const float* partial, void* out, int M, int N, int split_k,
                            int epilogue, const SmallFuse& fuse);

// ---- small-M variant (M <= 32: decode batches) --------------------------------------------------
// Same operand mapping, a schedule built around two facts measured on this part:
// (1) the weight stream only stays pipelined if every vector-memory load sits at
// a fixed place in a branch-free loop body -- then the compiler can wait with an
// exact s_waitcnt vmcnt(n); a branch around a load makes it wait for everything,
// and without a scheduling barrier it sinks the ring reloads to the end of the
// body; (2) with 13 VALU ops per packed word the kernel is close to VALU-bound,
// so nothing else may cost vector instructions (addresses are scalar base + a
// fixed lane offset, per-group constants arrive precomputed from LDS).
//
// K is walked in stages of 8 steps (256 k).  While a stage is consumed, the
// activations and per-group constants of the next one travel global -> registers
// -> the other LDS buffer; one barrier per stage.  The ring keeps 8 KiB of
// weights per wave in flight at all times.
constexpr int kSmallDepth = 8;  // steps per stage = ring depth

// NORM: x is the element-wise half of an RMSNorm, fp16(h * norm_w), written by the
// producer of h (kEpilogueResidual); the row factor 1 / sqrt(ssq[m] / K + eps), with
// ssq[m] the sum of the fuse.ssq_tiles partial sums of squares the producer left
// behind, scales the fp32 accumulators at the end, so the row never needs a pass
// of its own.
// STREAM: the balanced plan described below (it costs registers: a second set of
// accumulators), otherwise only the regular one.
// KW: K shares inside the workgroup.  With KW = 2 the workgroup has eight waves, two sets of four that
// walk consecutive K ranges of the same column tile, each with its own staged activations and constants,
// and add their sums through LDS at the end: where the column tiles alone nearly fill the GPU (one
// workgroup per CU, two waves per SIMD) a tile then needs no partial sums from another workgroup, so up
// to 32 rows finish -- epilogue included -- inside the launch, without a second stage.
template <int BITS, int MT, int SPG, bool NORM, bool STREAM, int KW = 1>
__global__ __launch_bounds__(256 * KW) void gptq_gemm_small_kernel(
    const half_t* __restrict__ x_all, const uint32_t* __restrict__ qweight,
    const uint32_t* __restrict__ qzeros, const half_t* __restrict__ scales,
    half_t* out_all, float* partial_all, unsigned* counters,
    int M_all, int N, int K, int steps_total, int stages_per_block, int split_k, int stream_units, int epilogue,
    SmallFuse fuse) {
    constexpr int P = Packing<BITS>::kPerWord;
    constexpr int PAIRS = Packing<BITS>::kPairs;
    constexpr uint32_t MASK = Packing<BITS>::kMask;
    constexpr int ROWS_PER_STEP = 32 / P;
    constexpr int LOADS = ROWS_PER_STEP / 4;
    constexpr int D = kSmallDepth;
    constexpr int GPS = D / SPG;            // groups per stage
    constexpr int BM = 16 * MT;
    // More rows than one workgroup takes: blockIdx.z picks a block of BM rows (regular
    // plan, no in-kernel reduction).  The row blocks read the same packed weights at
    // the same time, so one of them finds them in a cache; the partial sums of all
    // blocks form one [split][M_all][N] array for the second stage.
    const int row0 = blockIdx.z * BM;
    const int M = min(M_all - row0, BM);
    const half_t* __restrict__ x = x_all + (size_t)row0 * K;
    half_t* out = out_all + (size_t)row0 * N;
    float* partial = partial_all + (size_t)row0 * N;
    const size_t plane = (size_t)M_all * N;  // one split's partial sums
    constexpr int XCH = D * 4;              // 16-byte activation chunks per row per stage
    constexpr int RS = XCH + 1;             // padded row stride
    constexpr int XL = BM * XCH / 256;      // chunks each thread stages: 2 (MT=1) or 4 (MT=2)
    static_assert(D % SPG == 0, "a stage must hold whole groups");

    static_assert(KW == 1 || (KW == 2 && !STREAM), "one or two K shares; the balanced plan has one");
    constexpr int NT = 256 * KW;  // threads of the workgroup
    __shared__ uint4 xs_all[2][KW][BM * RS];
    __shared__ uint32_t cs_all[2][KW][GPS][3][kGemmCols];  // scale pair, zero_lo pair, zero_hi pair
    __shared__ float inv_rms_s[NORM ? BM : 1];

    const int wg_tid = threadIdx.x;                                            // 0 .. NT - 1: results and epilogues
    const int kh = KW == 1 ? 0 : __builtin_amdgcn_readfirstlane(wg_tid >> 8);  // this thread's K share
    const int tid = wg_tid & 255;                                              // within the share: loop and staging
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nl = lane & 15, kq = lane >> 4;
    const int lcol = wave * 64 + nl * 4;
    const int last_step = steps_total - 1;
    const int g_last = last_step / SPG;

    // The work of a workgroup is stages_per_block consecutive stages of a walk over
    // (column tile, stage) pairs, tile by tile.  Regular plan (stream_units == 0):
    // grid (tiles, splits), a workgroup stays inside its tile.  Balanced plan: 1-D
    // grid over a walk with stream_units stages per tile, cut into equal ranges; a
    // range may end one tile and begin the next (n0 stages of tile t0 from stage
    // s0, then n1 stages of tile t0 + 1 from its stage 0).  The K loop runs through
    // both without a break; the first tile's accumulators are set aside at the
    // border.  A tile's contributors are consecutive workgroups, which gives each
    // its slot among the partial sums and every tile its count.
    int t0, s0, n0, n1, slot0, nseg0, nseg1;
    if (!STREAM || stream_units == 0) {
        t0 = blockIdx.x;
        s0 = (blockIdx.y * KW + kh) * stages_per_block;  // the shares of a workgroup walk consecutive ranges
        n0 = stages_per_block;
        n1 = 0;
        slot0 = blockIdx.y;
        nseg0 = split_k;
        nseg1 = 0;
    } else {
        const int S = stream_units, q = stages_per_block;
        const int lo = blockIdx.x * q, hi = min(lo + q, (N + kGemmCols - 1) / kGemmCols * S);
        t0 = lo / S;
        s0 = lo - t0 * S;
        n0 = min(S - s0, hi - lo);
        n1 = hi - lo - n0;
        slot0 = blockIdx.x - t0 * S / q;
        nseg0 = (t0 * S + S - 1) / q - t0 * S / q + 1;
        nseg1 = ((t0 + 1) * S + S - 1) / q - (t0 + 1) * S / q + 1;  // this workgroup holds slot 0 there
    }
    const int n_stages = n0 + n1;
    // stage i of the range: its tile and its first step within K
    auto tile_of = [&](int i) { return i < n0 ? t0 : t0 + 1; };
    auto step_of = [&](int i) { return (i < n0 ? s0 + i : i - n0) * D; };

    // ---- weight ring
    uint4_t qb[D][LOADS];
    uint32_t lane_off[LOADS];
#pragma unroll
    for (int j = 0; j < LOADS; ++j) lane_off[j] = (uint32_t)((kq * LOADS + j) * N + lcol) * 4u;
    // Buffer loads: the scalar offset of the step and the lane's fixed 32-bit offset
    // go to the instruction as they are (no vector address arithmetic, and measured
    // 3-4 % faster than global_load with a 64-bit address pair on the large shapes);
    // streaming hint, agent scope: every packed word is read once.  The tile's first
    // column travels in the scalar offset; columns past N (last tile) read the
    // neighbouring row or, past the end of the buffer, zero, and are never stored.
    const __amdgpu_buffer_rsrc_t q_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(qweight), 0, (int)((size_t)(K / P) * N * 4), kBufferRsrcFlags);
    // The ring is refilled at a fixed place of the loop body, also in the range's last
    // stage, where nothing is left to fetch: those loads go through a descriptor of
    // zero records, so they return zero without touching memory.
    const __amdgpu_buffer_rsrc_t q_none =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(qweight), 0, 0, kBufferRsrcFlags);
    auto load_q = [&](const __amdgpu_buffer_rsrc_t& rsrc, int tile, int step, uint4_t* dst) {
        const int s = min(step, last_step);
        const int soff = (s * ROWS_PER_STEP * N + tile * kGemmCols) * 4;
#pragma unroll
        for (int j = 0; j < LOADS; ++j)
            dst[j] = __builtin_bit_cast(
                uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)lane_off[j], soff, kBufferStreamAgent));
    };
    // NORM, two row tiles: the producer's sums of squares are requested ahead of the ring -- loads
    // return in order, and behind the ring's 8 KiB per wave (and in three dependent steps) they kept
    // the first stage waiting until long after the whole ring had landed; they are summed after the
    // first stage's loads have been issued (decode at batch 32: 17.06 -> 16.88 ms per token).  With
    // one row tile the same order measured slower (batch 1: 8.89 -> 8.97 ms), so there they stay
    // behind the ring.
    constexpr bool SSQ_AHEAD = NORM && MT == 2;
    constexpr int SSQ_PASSES = NORM ? (BM * 32 + 255) / 256 : 1;
    SsqLane ssq_pre[SSQ_AHEAD ? SSQ_PASSES : 1];
    if constexpr (SSQ_AHEAD) {
#pragma unroll
        for (int pass = 0; pass < SSQ_PASSES; ++pass) {
            const int row = min(pass * 8 + ((wg_tid & 255) >> 5), M - 1);
            ssq_pre[pass] = ssq_lane_load(fuse.ssq_in + (size_t)row * fuse.ssq_tiles, fuse.ssq_tiles, wg_tid & 31);
        }
        __builtin_amdgcn_sched_barrier(0);  // ahead of the ring, not among or behind its loads
    }
#pragma unroll
    for (int d = 0; d < D; ++d) load_q(q_rsrc, t0, s0 * D + d, qb[d]);

    // ---- staging of activations and constants: global -> registers -> LDS
    uint4 xr[XL];
    // Constants of a stage: GPS groups x 256 columns, CE adjacent columns of one
    // group per thread, so that every wave runs the same (short) instruction
    // sequence -- a wave pays for an instruction whatever the number of live lanes.
    constexpr int CE = GPS;                    // 1, 2, 4 or 8
    constexpr int CT = kGemmCols / CE;         // threads per group
    constexpr int ZW = CE > P ? CE / P : 1;    // packed zero words per thread
    uint32_t sr[(CE + 1) / 2];                 // CE scales
    uint32_t zr[ZW];
    int x_row[XL], x_chunk[XL];
#pragma unroll
    for (int u = 0; u < XL; ++u) {
        const int idx = u * 256 + tid;
        x_row[u] = min(idx / XCH, M - 1);  // rows >= M only feed accumulator rows that are never stored
        x_chunk[u] = idx % XCH;
    }
    const int c_group = tid / CT, c_col0 = tid % CT * CE;
    // Buffer loads again: a fixed per-thread offset plus a scalar one that carries the
    // stage (group row, k) and the tile, so that moving on to the next stage or tile
    // costs no vector arithmetic.  Columns past N pick up the next row's values or,
    // past the end, zero: they only feed columns that are never stored.
    const __amdgpu_buffer_rsrc_t x_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(x), 0, (int)((size_t)M * K * 2), kBufferRsrcFlags);
    const __amdgpu_buffer_rsrc_t s_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<half_t*>(scales), 0, (int)((size_t)(g_last + 1) * N * 2), kBufferRsrcFlags);
    const __amdgpu_buffer_rsrc_t z_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(qzeros), 0, (int)((size_t)(g_last + 1) * (N / P) * 4), kBufferRsrcFlags);
    int x_off[XL];
#pragma unroll
    for (int u = 0; u < XL; ++u) x_off[u] = (x_row[u] * K + x_chunk[u] * 8) * 2;
    const int s_off = (c_group * N + c_col0) * 2, z_off = (c_group * (N / P) + c_col0 / P) * 4;
    auto fetch_stage = [&](int i) {
        const int sclamp = min(step_of(i), (last_step / D) * D);  // never read past K
        const int g0 = sclamp / SPG, tile = tile_of(i);  // groups past the last one (dead steps) read zero
#pragma unroll
        for (int u = 0; u < XL; ++u)
            xr[u] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, x_off[u], sclamp * 64, 0));
        const int s_soff = (g0 * N + tile * kGemmCols) * 2;
        if constexpr (CE == 1) {
            sr[0] = __builtin_amdgcn_raw_buffer_load_b16(s_rsrc, s_off, s_soff, 0);
        } else if constexpr (CE == 2) {
            sr[0] = __builtin_amdgcn_raw_buffer_load_b32(s_rsrc, s_off, s_soff, 0);
        } else if constexpr (CE == 4) {
            const uint2_t v = __builtin_bit_cast(uint2_t, __builtin_amdgcn_raw_buffer_load_b64(s_rsrc, s_off, s_soff, 0));
            sr[0] = v[0];
            sr[1] = v[1];
        } else {
            const uint4_t v = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(s_rsrc, s_off, s_soff, 0));
#pragma unroll
            for (int j = 0; j < 4; ++j) sr[j] = v[j];
        }
        const int z_soff = (g0 * (N / P) + tile * (kGemmCols / P)) * 4;
#pragma unroll
        for (int j = 0; j < ZW; ++j) zr[j] = __builtin_amdgcn_raw_buffer_load_b32(z_rsrc, z_off + j * 4, z_soff, 0);
    };
    auto store_stage = [&](int buf, int i) {
        const int stage_step = step_of(i);
#pragma unroll
        for (int u = 0; u < XL; ++u) {
            const uint32_t in[4] = {xr[u].x, xr[u].y, xr[u].z, xr[u].w};
            uint32_t o[4];
            if constexpr (BITS == 4) {
                pair_activations<4>(in, o);
            } else {
                pair_activations<8>(in, o);
                pair_activations<8>(in + 2, o + 2);
            }
            // steps past the end of K contribute nothing
            const bool live = stage_step + x_chunk[u] / 4 <= last_step;
            xs_all[buf][kh][(u * 256 + tid) / XCH * RS + x_chunk[u]] =
                live ? make_uint4(o[0], o[1], o[2], o[3]) : make_uint4(0, 0, 0, 0);
        }
        {
            const int zsub = CE >= P ? 0 : c_col0 % P;  // first sub-word of this thread in zr[0]
            uint32_t k_scale[CE], k_lo[CE], k_hi[CE];
#pragma unroll
            for (int j = 0; j < CE; ++j) {
                const uint32_t z = (zr[j / P] >> ((zsub + j % P) * BITS)) & MASK;
                const uint32_t sbits = (sr[j / 2] >> (j % 2 * 16)) & 0xFFFFu;
                const ColumnConst k = column_const_from_bits(sbits, z);
                k_scale[j] = as_u32(k.scale);
                k_lo[j] = as_u32(k.zero_lo);
                k_hi[j] = as_u32(k.zero_hi);
            }
            struct alignas(CE * 4) ConstWords { uint32_t w[CE]; };
#pragma unroll
            for (int r = 0; r < 3; ++r) {
                const uint32_t* src = r == 0 ? k_scale : r == 1 ? k_lo : k_hi;
                ConstWords v;
#pragma unroll
                for (int j = 0; j < CE; ++j) v.w[j] = src[j];
                *reinterpret_cast<ConstWords*>(&cs_all[buf][kh][c_group][r][c_col0]) = v;
            }
        }
    };

    fetch_stage(0);
    if constexpr (NORM) {
        // 1 / rms of every row from the producer's per-tile sums of squares: 32
        // lanes per row read the tiles in parallel (the loads travel with those of
        // the first stage) and are folded by shuffles, a fixed order; read back
        // after the K loop
#pragma unroll
        for (int pass = 0; pass < SSQ_PASSES; ++pass) {
            const int row = pass * 8 + (tid >> 5), p0 = tid & 31;
            float ss = 0.f;
            if (row < M) {
                const float* pieces = fuse.ssq_in + (size_t)row * fuse.ssq_tiles;
                if constexpr (SSQ_AHEAD)
                    ss = ssq_lane_sum(ssq_pre[pass], pieces, fuse.ssq_tiles, p0);
                else
                    ss = ssq_lane_sum(ssq_lane_load(pieces, fuse.ssq_tiles, p0), pieces, fuse.ssq_tiles, p0);
            }
#pragma unroll
            for (int off = 1; off < 32; off <<= 1) ss += __shfl_xor(ss, off);
            if (p0 == 0 && row < BM && kh == 0) inv_rms_s[row] = 1.f / sqrtf(ss / (float)K + fuse.eps);
        }
    }
    store_stage(0, 0);
    fetch_stage(1);
    __syncthreads();

    DequantRegs regs;
    regs.init(BITS);
    float4_t acc[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[mt][t] = float4_t{0.f, 0.f, 0.f, 0.f};
    float4_t acc_first[STREAM ? MT : 1][4];  // the first tile's sums when the range goes on into a second tile
#pragma unroll
    for (int mt = 0; mt < (STREAM ? MT : 1); ++mt)
#pragma unroll
        for (int t = 0; t < 4; ++t) acc_first[mt][t] = float4_t{0.f, 0.f, 0.f, 0.f};
    ColumnConst cc[4];

    for (int stage = 0; stage < n_stages; ++stage) {
        const int buf = stage & 1;
        // Two workgroups share a CU on most plans, and the older one wins every arbitration: it runs
        // ahead and leaves the younger one to finish alone, with half the CU's loads in flight
        // (8192 x 57344 at one row: the first 256 workgroups leave the loop 13 us before the other
        // 256).  The priority of a wave falls with its progress through its range, in four steps, so
        // whichever workgroup is behind is served first (46.4 -> 45.2 us for that launch).
        if constexpr (KW == 1) {
            // (balanced plan: the workgroups of the second half of the grid are the younger ones of their
            // CUs; they step down an eighth of the range later, which halves the lead the older one can
            // take: 46.3 -> 45.3 us more.  On the two-dimensional grids the same offset measured slower.)
            const int late = (STREAM && stream_units != 0 && blockIdx.x * 2 >= gridDim.x) ? n_stages : 0;  // in eighths of a stage
            set_priority_by_progress(stage, n_stages, late);
        }
        const int next_tile = tile_of(stage + 1), next_step = step_of(stage + 1);
        const __amdgpu_buffer_rsrc_t next_rsrc = stage + 1 < n_stages ? q_rsrc : q_none;
#pragma unroll
        for (int d = 0; d < D; ++d) {
            if (d % SPG == 0) {  // compile-time: a new group starts here
                const uint4 sc4 = *reinterpret_cast<const uint4*>(&cs_all[buf][kh][d / SPG][0][lcol]);
                const uint4 lo4 = *reinterpret_cast<const uint4*>(&cs_all[buf][kh][d / SPG][1][lcol]);
                const uint4 hi4 = *reinterpret_cast<const uint4*>(&cs_all[buf][kh][d / SPG][2][lcol]);
                cc[0] = ColumnConst{as_half2(sc4.x), as_half2(lo4.x), as_half2(hi4.x)};
                cc[1] = ColumnConst{as_half2(sc4.y), as_half2(lo4.y), as_half2(hi4.y)};
                cc[2] = ColumnConst{as_half2(sc4.z), as_half2(lo4.z), as_half2(hi4.z)};
                cc[3] = ColumnConst{as_half2(sc4.w), as_half2(lo4.w), as_half2(hi4.w)};
            }
            half8_t b[4];
            uint4_t* q = qb[d];
            const uint32_t qa[4] = {q[0].x, q[0].y, q[0].z, q[0].w};
            const uint32_t qc[4] = {q[LOADS - 1].x, q[LOADS - 1].y, q[LOADS - 1].z, q[LOADS - 1].w};
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                half2_t w[4];
                dequant_word<BITS>(qa[t], cc[t], regs, w);
                if constexpr (BITS == 8) dequant_word<BITS>(qc[t], cc[t], regs, w + PAIRS);
                const uint4_t packed = {as_u32(w[0]), as_u32(w[1]), as_u32(w[2]), as_u32(w[3])};
                b[t] = __builtin_bit_cast(half8_t, packed);
            }
            load_q(next_rsrc, next_tile, next_step + d, q);
            __builtin_amdgcn_sched_barrier(0);  // keep the reload here (see above)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const half8_t a = __builtin_bit_cast(half8_t, xs_all[buf][kh][(mt * 16 + nl) * RS + d * 4 + kq]);
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b[t], acc[mt][t], 0, 0, 0);
            }
        }
        store_stage(buf ^ 1, stage + 1);
        fetch_stage(stage + 2);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        if (STREAM && stage == n0 - 1 && n1 > 0) {  // border between the two tiles: registers only
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    acc_first[mt][t] = acc[mt][t];
                    acc[mt][t] = float4_t{0.f, 0.f, 0.f, 0.f};
                }
        }
    }

    if constexpr (KW == 2) {
        // the second share's sums go through LDS (the staging area, no longer read) to the first one, which
        // from here on is the workgroup: accumulator (mt, t) of lane `tid` at [(mt * 4 + t) * 256 + tid]
        static_assert(sizeof(xs_all) >= (size_t)MT * 4 * 256 * sizeof(float4_t), "staging area too small for the sums");
        float4_t* red = reinterpret_cast<float4_t*>(&xs_all[0][0][0]);
        __syncthreads();
        if (kh == 1) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int t = 0; t < 4; ++t) red[(mt * 4 + t) * 256 + tid] = acc[mt][t];
        }
        __syncthreads();
        if (kh == 0) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int t = 0; t < 4; ++t) acc[mt][t] += red[(mt * 4 + t) * 256 + tid];
        }
    }

    // Sums of a finished tile -> results, with the epilogue.  The sums are the splits' partial sums in
    // the workspace, added here in slot order, or (lds_tile != nullptr: a tile with a single contributor
    // whose sums never left the workgroup) one fp32 tile [BM][kGemmCols] in LDS.
    auto reduce_tile = [&](int tile, int nseg, const float* lds_tile) {
        constexpr int BATCH = 16;  // partial loads in flight per thread
        auto sum_splits = [&](const float* p) {
            if (lds_tile != nullptr) {  // p - partial = m * N + column: the tile's own column from LDS
                const size_t off = (size_t)(p - partial);
                return *reinterpret_cast<const float4_t*>(lds_tile + (off / N) * kGemmCols + (off % N - (size_t)tile * kGemmCols));
            }
            float4_t s = {0.f, 0.f, 0.f, 0.f};
            for (int sp = 0; sp < nseg; sp += BATCH) {
                float4_t v[BATCH];
#pragma unroll
                for (int u = 0; u < BATCH; ++u)
                    v[u] = sp + u < nseg ? load_agent4(p + (size_t)(sp + u) * plane) : float4_t{0.f, 0.f, 0.f, 0.f};
                wait_agent_loads(v);
#pragma unroll
                for (int u = 0; u < BATCH; ++u)
                    if (sp + u < nseg) s += v[u];
            }
            return s;
        };
        // two runs of partials (same slots), requested together: one wait instead of two
        auto sum_splits2 = [&](const float* p, const float* q, float4_t& a, float4_t& b) {
            if (lds_tile != nullptr) {
                a = sum_splits(p);
                b = sum_splits(q);
                return;
            }
            constexpr int HALF = BATCH / 2;
            a = float4_t{0.f, 0.f, 0.f, 0.f};
            b = a;
            for (int sp = 0; sp < nseg; sp += HALF) {
                float4_t v[BATCH];
#pragma unroll
                for (int u = 0; u < HALF; ++u) {
                    const bool live = sp + u < nseg;
                    v[u] = live ? load_agent4(p + (size_t)(sp + u) * plane) : float4_t{0.f, 0.f, 0.f, 0.f};
                    v[HALF + u] = live ? load_agent4(q + (size_t)(sp + u) * plane) : float4_t{0.f, 0.f, 0.f, 0.f};
                }
                wait_agent_loads(v);
#pragma unroll
                for (int u = 0; u < HALF; ++u)
                    if (sp + u < nseg) {
                        a += v[u];
                        b += v[HALF + u];
                    }
            }
        };
        if (epilogue == kEpilogueSiluPairs) {
            // columns [0, 128) of the tile are gate, [128, 256) the matching up columns
            for (int item = wg_tid; item < M * (kGemmCols / 8); item += NT) {
                const int m = item / (kGemmCols / 8), c4 = item % (kGemmCols / 8) * 4;
                const float* p = partial + (size_t)m * N + tile * kGemmCols + c4;
                float4_t g, u;
                sum_splits2(p, p + kGemmCols / 2, g, u);
                half4_t gh = {(half_t)g[0], (half_t)g[1], (half_t)g[2], (half_t)g[3]};
                half4_t uh = {(half_t)u[0], (half_t)u[1], (half_t)u[2], (half_t)u[3]};
                if (fuse.bias) {  // the bias of the gate and of the up projection, before the activation
                    gh = gh + *reinterpret_cast<const half4_t*>(fuse.bias + tile * kGemmCols + c4);
                    uh = uh + *reinterpret_cast<const half4_t*>(fuse.bias + tile * kGemmCols + kGemmCols / 2 + c4);
                }
                half4_t h;
#pragma unroll
                for (int e = 0; e < 4; ++e) h[e] = silu_pair(gh[e], uh[e]);
                *reinterpret_cast<half4_t*>(out + (size_t)m * (N / 2) + tile * (kGemmCols / 2) + c4) = h;
            }
            return;
        }
        if (epilogue == kEpilogueRopeAppend) {
            // four consecutive columns = two interleaved pairs of one head
            for (int item = wg_tid; item < M * (kGemmCols / 4); item += NT) {
                const int m = item / (kGemmCols / 4), c = tile * kGemmCols + item % (kGemmCols / 4) * 4;
                // the row's position and its cos/sin are requested before the partials,
                // whose wait then covers them
                const int head = c / 128, d = c % 128;
                const int pos = min(max(fuse.positions[m], 0), fuse.max_seq - 1);
                const bool rotated = head < fuse.q_heads + fuse.kv_heads;
                float cr[2] = {0.f, 0.f}, sr[2] = {0.f, 0.f};
                if (rotated) {
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        cr[j] = fuse.rope_cos[(size_t)pos * 64 + d / 2 + j];
                        sr[j] = fuse.rope_sin[(size_t)pos * 64 + d / 2 + j];
                    }
                }
                const float4_t sum = sum_splits(partial + (size_t)m * N + c);
                half4_t y = {(half_t)sum[0], (half_t)sum[1], (half_t)sum[2], (half_t)sum[3]};
                if (fuse.bias) y = y + *reinterpret_cast<const half4_t*>(fuse.bias + c);
                if (!rotated) {  // value head: copied, cache is tiled
                    half_t* dst = fuse.vt_cache + ((size_t)m * fuse.kv_heads + (head - fuse.q_heads - fuse.kv_heads)) * 128 * fuse.max_seq +
                                  vt_offset(d, pos);
#pragma unroll
                    for (int e = 0; e < 4; ++e) dst[e * kVTile] = y[e];
                    continue;
                }
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
            return;
        }
        if (epilogue == kEpilogueResidual) {
            // a wave owns one row of the tile per pass (64 lanes x 4 columns), so the
            // row's sum of squares is one wave reduction; N is a multiple of 256
            for (int base = 0; base < M * (kGemmCols / 4); base += NT) {
                const int m = base / (kGemmCols / 4) + (wg_tid >> 6), c = tile * kGemmCols + lane * 4;
                float ss = 0.f;
                if (m < M) {
                    // the old value of the stream and the next norm's weight are requested
                    // before the partials, whose wait then covers them
                    half_t* hp = out + (size_t)m * N + c;
                    const half4_t h_old = *reinterpret_cast<const half4_t*>(hp);
                    half4_t nw = {(half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f};
                    if (fuse.xw_out) nw = *reinterpret_cast<const half4_t*>(fuse.next_norm_w + c);
                    const float4_t s = sum_splits(partial + (size_t)m * N + c);
                    half4_t y = {(half_t)s[0], (half_t)s[1], (half_t)s[2], (half_t)s[3]};
                    if (fuse.bias) y = y + *reinterpret_cast<const half4_t*>(fuse.bias + c);
                    const half4_t h = h_old + y;  // fp16 add, one rounding
                    *reinterpret_cast<half4_t*>(hp) = h;
                    if (fuse.xw_out) *reinterpret_cast<half4_t*>(fuse.xw_out + (size_t)m * N + c) = norm_weighted(h, nw, fuse.xw_clamped);
#pragma unroll
                    for (int e = 0; e < 4; ++e) ss += (float)h[e] * (float)h[e];
                }
                ss = wave_sum(ss);
                if (lane == 0 && m < M) fuse.ssq_out[(size_t)m * (N / kGemmCols) + tile] = ss;
            }
            return;
        }
        for (int item = wg_tid; item < M * (kGemmCols / 4); item += NT) {
            const int m = item / (kGemmCols / 4), c = tile * kGemmCols + item % (kGemmCols / 4) * 4;
            if (c >= N) continue;
            const float4_t s = sum_splits(partial + (size_t)m * N + c);
            half4_t h = {(half_t)s[0], (half_t)s[1], (half_t)s[2], (half_t)s[3]};
            if (fuse.bias) h = h + *reinterpret_cast<const half4_t*>(fuse.bias + c);
            *reinterpret_cast<half4_t*>(out + (size_t)m * N + c) = h;
        }
    };
    if constexpr (KW == 2) {
        if (counters != nullptr && epilogue != kEpilogueNone) {
            // two shares, K not split over workgroups: this workgroup holds the tile's finished sums, and the
            // epilogue reads them from LDS instead of from partial sums published to memory
            float* tile_s = reinterpret_cast<float*>(&xs_all[0][0][0]);
            static_assert(sizeof(xs_all) >= (size_t)BM * kGemmCols * sizeof(float), "staging area too small for the tile");
            __syncthreads();  // the sums of the second share have been read
            if (kh == 0) {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int m = mt * 16 + kq * 4 + r;
                        if (m >= M) continue;
                        float4_t v = {acc[mt][0][r], acc[mt][1][r], acc[mt][2][r], acc[mt][3][r]};
                        if constexpr (NORM) v *= inv_rms_s[m];
                        *reinterpret_cast<float4_t*>(tile_s + m * kGemmCols + lcol) = v;
                    }
            }
            __syncthreads();
            reduce_tile(t0, 1, tile_s);
            return;
        }
    }

    // ---- results.  A tile with several contributors: every one publishes its
    // fp32 partial tile with agent-scope stores (they go through to memory, which
    // is what workgroups on other XCDs see) and counts itself in; the one that
    // arrives last adds the partials in slot order -- a fixed order, so the result
    // does not depend on which workgroup that is -- and puts the counter back to
    // zero for the next launch.  The SiLU-pair, residual and RoPE epilogues always
    // take this route (they need the whole tile).  A workgroup that worked on two
    // tiles publishes both, waits once, and may be the last one of either.
    const int n_seg = STREAM && n1 > 0 ? 2 : 1;
    __shared__ int is_last[2];
    bool need_reduce = false;
    for (int sg = 0; sg < n_seg; ++sg) {
        const int tile = t0 + sg, slot = sg == 0 ? slot0 : 0, nseg = sg == 0 ? nseg0 : nseg1;
        const int col = tile * kGemmCols + lcol;
        const bool first_of_two = STREAM && sg == 0 && n1 > 0;
        const bool direct = nseg == 1 && epilogue == kEpilogueNone;
        need_reduce = need_reduce || !direct;
        if (col >= N || kh != 0) continue;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = mt * 16 + kq * 4 + r;
                if (m >= M) continue;
                float4_t v;
#pragma unroll
                for (int t = 0; t < 4; ++t) v[t] = first_of_two ? acc_first[STREAM ? mt : 0][t][r] : acc[mt][t][r];
                if constexpr (NORM) v *= inv_rms_s[m];
                if (direct) {
                    half4_t h = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
                    if (fuse.bias) h = h + *reinterpret_cast<const half4_t*>(fuse.bias + col);
                    *reinterpret_cast<half4_t*>(out + (size_t)m * N + col) = h;
                } else {
                    float* dst = partial + (size_t)slot * plane + (size_t)m * N + col;
                    if (counters)
                        store_agent4(dst, v);
                    else
                        *reinterpret_cast<float4_t*>(dst) = v;
                }
            }
    }
    if (!need_reduce || counters == nullptr) return;  // without counters a second kernel adds the partials

    // every thread's stores acknowledged, then one arrival per tile
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    // (a workgroup that worked on two tiles counts in at both at once, from two waves: one after the
    // other the two round trips are 1.5 us of the launch's tail)
    if ((wg_tid & 63) == 0 && (wg_tid >> 6) < n_seg) {
        const int sg = wg_tid >> 6;
        const unsigned expected = sg == 0 ? nseg0 : nseg1;
        int last = 0;
        if (!(expected == 1 && epilogue == kEpilogueNone)) {
            const unsigned prev =
                __hip_atomic_fetch_add(&counters[t0 + sg], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last = prev == expected - 1;
            if (last) __hip_atomic_store(&counters[t0 + sg], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        is_last[sg] = last;
    }
    __syncthreads();

    for (int sg = 0; sg < n_seg; ++sg)
        if (is_last[sg]) reduce_tile(t0 + sg, sg == 0 ? nseg0 : nseg1, nullptr);
}

// gptq_gemm_cols.hip
bool gemm_cols_preferred(int M, int N, int K, int group_size, int bits, int epilogue);
size_t gemm_cols_workspace_bytes(int M, int N, int K);
int gptq_gemm_cols_launch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                          const void* scales, void* out, int M, int N, int K, int group_size, int bits, int epilogue,
                          const SmallFuse& fuse, void* workspace, size_t workspace_bytes);

// gptq_gemm_wide.hip: more than 64 rows, dequantised weight tiles staged in LDS
bool gemm_wide_preferred(int M, int N, int K, int group_size, int bits, int epilogue);
size_t gemm_wide_workspace_bytes(int M, int N, int K);
int gptq_gemm_wide_launch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                          const void* scales, void* out, int M, int N, int K, int group_size, void* workspace,
                          size_t workspace_bytes, const half_t* bias);

// gptq_gemm_tall.hip: blocks of 128 rows, weights dequantised in registers, K sliced over the waves
bool gemm_tall_preferred(int M, int N, int K, int group_size, int bits, int epilogue);
size_t gemm_tall_workspace_bytes(int M, int N, int K);
bool gemm_tall_silu_pairs_supported(int M, int N, int K, int group_size, int bits);
int gptq_gemm_tall_launch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                          const void* scales, void* out, int M, int N, int K, int group_size, void* workspace,
                          size_t workspace_bytes, const half_t* bias, int epilogue);

struct GemmPlan {
    int mt;  // 16-row tiles per block: 1, 2, 4 or 8
    int col_tiles;
    int m_blocks;
    int split_k;  // partial-sum slots per tile
    int steps_total;
    int steps_per_block;
    int stream_units = 0;  // small-M kernel, balanced plan: stages per tile of the walk (0: regular plan)
    int blocks = 0;        // balanced plan: workgroups
    int k_ways = 1;        // small-M kernel: K shares inside a workgroup (2: eight waves, sums meet in LDS)
};

static int env_int_gemm(const char* name, int fallback) {
    const char* v = getenv(name);
    if (!v || !*v) return fallback;
    return atoi(v);
}

constexpr int kSmallMaxM = 32;     // rows of one launch with epilogues / norm fusion
constexpr int kSmallBlockM = 64;   // rows per pass of a plain product above kSmallMaxM rows
// (an A/B switch; workspace sizes and the row-blocked path assume at most kSmallMaxM)
static const int kFusedReduceMaxM = [] {
    const int v = env_int_gemm("MH_GEMM_FUSED_REDUCE_MAX_M", 8);
    return v < 1 ? 1 : v > kSmallMaxM ? kSmallMaxM : v;
}();

// Plan of the small-M kernel: column tiles x K splits sized so the GPU holds
// about MH_GEMM_SMALL_WAVES_PER_CU waves per CU; a block walks whole stages.
// GemmPlan::steps_per_block carries stages_per_block * kSmallDepth.
// Two K shares inside a workgroup of eight waves (KW = 2 of the kernel), K not split over workgroups: taken
// where the column tiles alone fill three quarters of the CUs or more (gate|up of the 70B shape: 224 tiles
// on 256 CUs) above the rows whose split-K sums the last workgroup of a tile adds cheaply -- from there on
// the fp32 partial sums of a split plan and their second stage cost more than the CUs left idle
// (8192 x 57344 at 32 rows: 14.7 MB of partial sums each way and a launch).  MH_GEMM_SMALL_KW (read at every
// call): 2 takes it for every row count it serves, 1 never.
static bool small_two_shares(int M, int N, int K, int group_size, int row_blocks, int bits) {
    // (groups of 32 would need 98 KiB of staged constants for the two shares)
    if (row_blocks != 1 || M > kSmallMaxM || group_size < 64) return false;
    const int tiles = (N + kGemmCols - 1) / kGemmCols, cus = compute_units();
    const long stages_total = (K / 32 + kSmallDepth - 1) / kSmallDepth;
    if (tiles > cus || 4 * tiles < 3 * cus || stages_total < 2 || tiles > kMaxTileCounters) return false;
    const char* v = getenv("MH_GEMM_SMALL_KW");
    if (v && *v) return atoi(v) == 2;
    // (8-bit weights at any row count: 8192 x 57344 at 1 / 4 / 8 rows 72.8 / 73.2 / 73.5 us against 77.1-78.5 /
    // 78.3 / 79.8 on the balanced plan; 4-bit weights at 8 rows 51.0 against 49.1)
    return M > kFusedReduceMaxM || bits == 8;
}

GemmPlan plan_gemm_small(int M, int N, int K, bool allow_balanced, int row_blocks = 1, int group_size = 128, int bits = 4) {
    GemmPlan p;
    p.mt = M <= 16 ? 1 : M <= 32 ? 2 : 4;
    p.col_tiles = (N + kGemmCols - 1) / kGemmCols;
    p.m_blocks = row_blocks;
    p.steps_total = K / 32;
    const long stages_total = (p.steps_total + kSmallDepth - 1) / kSmallDepth;
    if (small_two_shares(M, N, K, group_size, row_blocks, bits)) {
        p.k_ways = 2;
        p.split_k = 1;
        p.steps_per_block = (int)((stages_total + 1) / 2 * kSmallDepth);  // stages of one share
        return p;
    }
    static const int waves_per_cu = env_int_gemm("MH_GEMM_SMALL_WAVES_PER_CU", 8);
    const long target_blocks = (long)compute_units() * waves_per_cu / 4;
    long split = target_blocks / ((long)p.col_tiles * row_blocks);
    if (split > stages_total) split = stages_total;
    // fp32 partials cost 8*M*N bytes per split against K*N/2 bytes of weights
    // (a single block of more than 32 rows is bound by instruction issue and by the
    // CUs left idle, and more splits are worth twice the partial-sum traffic:
    // 4096x14336 at 64 rows 32.8 -> 26.6 us; with two or more row blocks side by
    // side the CUs are taken and the looser cap loses, 38.5 -> 42.1 us at 128 rows)
    const long cap_unit = M > 32 && row_blocks == 1 ? 16L * M : 32L * M;
    const long traffic_cap = K / cap_unit > 1 ? K / cap_unit : 1;
    if (split > traffic_cap) split = traffic_cap;
    // a workgroup walks two stages or more: its first stage's round trips stand in front of any arithmetic
    // (11008 x 4096 at 2 / 8 / 12 rows, one stage per workgroup against two: 8 bit 18.1 / 20.8 / 18.4 us against
    // 14.0 / 15.3 / 14.7, 4 bit 14.0 / 15.5 / 14.8 against 13.1 / 14.4 / 13.1; at least three: 4096 x 12288 at 12
    // rows 12.6 -> 16.6 us)
    if (split > stages_total / 2) split = stages_total / 2;
    if (split < 1) split = 1;
    const long spb = (stages_total + split - 1) / split;
    p.steps_per_block = (int)(spb * kSmallDepth);
    p.split_k = (int)((stages_total + spb - 1) / spb);
    // Above the rows of the in-kernel reduction every split costs 8 M N bytes of partial sums through HBM
    // and the second stage reads them all: pairs of consecutive K ranges go to one workgroup of eight
    // waves (KW = 2), whose two sums meet in LDS, which halves both (8192x10240 at 32 rows: 8 -> 4 slots).
    // Measured (us, paired / not): 8192x10240 at 24 / 32 rows 21.0 / 22.5, 21.8 / 24.2 (equal below);
    // 28672x8192 at 9 / 16 / 17 rows 28.5 / 28.9, 29.4 / 30.9, 34.1 / 35.2 but 38.8 / 36.7 at 32 rows, where
    // two row tiles meet long K ranges and the eight waves' common barrier per stage costs more than the
    // partial sums saved: with two row tiles it is taken up to K = 16384.
    if (M > kFusedReduceMaxM && M <= kSmallMaxM && row_blocks == 1 && group_size >= 64 && p.split_k >= 2 &&
        p.split_k % 2 == 0 && (M <= 16 || K <= 16384)) {
        const char* v = getenv("MH_GEMM_SMALL_KW");
        if (!(v && *v && atoi(v) == 1)) {
            p.k_ways = 2;
            p.split_k /= 2;
        }
    }
    // Balanced plan (in-kernel reduction only): the tiles' stages form one walk that
    // is cut into target_blocks equal ranges, so every CU gets the same number of
    // stages even where tiles x splits does not divide by the CUs (224 tiles x 2
    // splits on 256 CUs: 1.75 workgroups per CU, two on most).  A range covers at
    // most two tiles, and no tile gets more contributors than the caps above allow.
    // Worth it for long ranges only (measured: 8192x57344, 14 stages per workgroup,
    // 50.0 -> 48.1 us; 8192x10240, 3 stages, 15.2 -> 16.2 us: the workgroups that
    // work on two tiles end with two hand-offs), and not with an epilogue in the
    // reduction or the norm prologue (the same gate|up product with both: 49.7 ->
    // 54.1 us), which is what allow_balanced says.
    static const int balance = env_int_gemm("MH_GEMM_BALANCE", 1);
    if (balance && allow_balanced && M <= kFusedReduceMaxM && p.col_tiles <= kMaxTileCounters) {
        const long units = (long)p.col_tiles * stages_total;
        long q = (units + target_blocks - 1) / target_blocks;
        const long cap = traffic_cap < stages_total ? traffic_cap : stages_total;  // contributors per tile
        const long q_min = (stages_total + cap - 1) / cap;
        if (q < q_min) q = q_min;
        if (q >= 8 && q <= stages_total && stages_total % q != 0) {
            p.stream_units = (int)stages_total;
            p.steps_per_block = (int)(q * kSmallDepth);
            p.blocks = (int)((units + q - 1) / q);
            p.split_k = (int)((stages_total + q - 1) / q + 1);
        }
    }
    return p;
}

static bool use_small(int M, int group_size) {
    static const int off = env_int_gemm("MH_GEMM_NO_SMALL", 0);
    const int spg = group_size / 32;
    return !off && M <= kSmallMaxM && (spg == 1 || spg == 2 || spg == 4 || spg == 8);
}

GemmPlan plan_gemm(int M, int N, int K, int group_size, bool allow_balanced, int bits) {
    if (use_small(M, group_size)) return plan_gemm_small(M, N, K, allow_balanced, 1, group_size, bits);
    GemmPlan p;
    p.mt = M <= 16 ? 1 : M <= 32 ? 2 : M <= 64 ? 4 : 8;
    const int bm = 16 * p.mt;
    const int sc = p.mt <= 2 ? 16 : (p.mt == 4 ? 8 : 4);
    p.col_tiles = (N + kGemmCols - 1) / kGemmCols;
    p.m_blocks = (M + bm - 1) / bm;
    p.steps_total = K / 32;
    static const int blocks_per_cu = env_int_gemm("MH_GEMM_BLOCKS_PER_CU", 2);
    const long target_blocks = (long)compute_units() * blocks_per_cu;
    long split = target_blocks / ((long)p.col_tiles * p.m_blocks);
    // every block walks whole stages; partial sums cost 8*M*N bytes per split
    long max_split = (p.steps_total + sc - 1) / sc;
    // fp32 partials cost 8*M*N bytes per split against K*N/2 bytes of weights:
    // keep them under about a quarter of the weight traffic
    const long traffic_cap = K / (64L * M) > 1 ? K / (64L * M) : 1;
    if (max_split > traffic_cap) max_split = traffic_cap;
    if (split > max_split) split = max_split;
    if (split < 1) split = 1;
    long spb = (p.steps_total + split - 1) / split;
    spb = (spb + sc - 1) / sc * sc;
    p.steps_per_block = (int)spb;
    p.split_k = (int)((p.steps_total + spb - 1) / spb);
    return p;
}

// The MFMA kernels address the packed weights of a matrix with 32-bit buffer offsets.
static bool packed_weights_addressable(int N, int K, int bits) { return (size_t)K * N * bits / 8 < ((size_t)1 << 31); }

bool gemm_supported(int M, int N, int K, int group_size, int bits) {
    return M >= 1 && (bits == 4 || bits == 8) && N % 8 == 0 && K % 32 == 0 && group_size % 32 == 0 &&
           K % group_size == 0 && packed_weights_addressable(N, K, bits);
}

// The epilogue out[m, j] = silu(y[m, gate(j)]) * y[m, up(j)] on column tiles laid out as
// 128 gate columns followed by their 128 up columns; served by the small-M kernel only.
bool gemm_silu_pairs_supported(int M, int N, int K, int group_size, int bits) {
    return gemm_supported(M, N, K, group_size, bits) && use_small(M, group_size) && N % kGemmCols == 0;
}

// Residual-add / RoPE epilogues and the normalise-while-staging prologue: the
// small-M kernel.  Up to kFusedReduceMaxM rows the epilogue runs in the kernel's own
// reduction (sums of squares per 256-column tile); above, in the second stage
// (per 1024 columns, so N must be a multiple of that).
bool gemm_norm_fusion_supported(int M, int N, int K, int group_size, int bits, int epilogue) {
    if (!gemm_supported(M, N, K, group_size, bits) || !use_small(M, group_size)) return false;
    if ((epilogue == kEpilogueResidual || epilogue == kEpilogueRopeAppend) &&
        gemm_cols_preferred(M, N, K, group_size, bits, epilogue))
        return true;
    if (M <= kFusedReduceMaxM || small_two_shares(M, N, K, group_size, 1, bits))
        return N % kGemmCols == 0 && (N + kGemmCols - 1) / kGemmCols <= kMaxTileCounters;
    return N % (epilogue == kEpilogueResidual ? 1024 : kGemmCols) == 0;
}

// The bias of a plain product (SmallFuse::bias) is added where the results are stored by every
// kernel except the staged one (group sizes other than 32 / 64 / 128 / 256).
bool gemm_bias_supported(int M, int N, int K, int group_size, int bits) {
    return gemm_supported(M, N, K, group_size, bits) &&
           (gemm_tall_preferred(M, N, K, group_size, bits, kEpilogueNone) ||
            gemm_wide_preferred(M, N, K, group_size, bits, kEpilogueNone) ||
            gemm_cols_preferred(M, N, K, group_size, bits, kEpilogueNone) ||
            use_small(M < kSmallMaxM ? M : kSmallMaxM, group_size));
}

// Per-row pieces a kEpilogueResidual producer leaves in ssq_out for this shape.
int gemm_residual_ssq_pieces(int M, int N, int K, int group_size, int bits) {
    if (gemm_cols_preferred(M, N, K, group_size, bits, kEpilogueResidual)) return N / 32;
    return M <= kFusedReduceMaxM || small_two_shares(M, N, K, group_size, 1, bits) ? N / kGemmCols : N / 1024;
}

static bool row_blocked(int M, int group_size) { return M > kSmallMaxM && use_small(kSmallMaxM, group_size); }

size_t gemm_workspace_bytes(int M, int N, int K, int group_size, int bits) {
    // Up to kSmallMaxM rows a launch with an epilogue or the norm prologue takes the small-M or the
    // column-owner kernel where the plain product takes the 128-row-block kernel: the size covers all three.
    const size_t tall = gemm_tall_preferred(M, N, K, group_size, bits, kEpilogueNone) ? gemm_tall_workspace_bytes(M, N, K) : 0;
    if (M > kSmallMaxM && gemm_tall_preferred(M, N, K, group_size, bits, kEpilogueNone)) return tall;
    if (gemm_wide_preferred(M, N, K, group_size, bits, kEpilogueNone)) return gemm_wide_workspace_bytes(M, N, K);
    if (row_blocked(M, group_size)) {
        // blocks of kSmallBlockM rows in one launch; partial sums [split][M][N]
        const GemmPlan p = plan_gemm_small(kSmallBlockM, N, K, false, (M + kSmallBlockM - 1) / kSmallBlockM);
        // unsplit, the kernel stores its results directly and touches neither counters nor partials
        return p.split_k > 1 ? kTileCounterBytes + (size_t)p.split_k * M * N * sizeof(float) : 0;
    }
    // either plan of the small-M kernel may be the one a launch takes
    const GemmPlan p = plan_gemm(M, N, K, group_size, false, bits), pb = plan_gemm(M, N, K, group_size, true, bits);
    const int slots = p.split_k > pb.split_k ? p.split_k : pb.split_k;
    // the small-M kernel may be asked for an epilogue that goes through the partials even unsplit
    if (slots <= 1 && !use_small(M, group_size)) return tall;
    const size_t small = kTileCounterBytes + (size_t)slots * M * N * sizeof(float);
    const size_t cols = M <= kSmallMaxM ? gemm_cols_workspace_bytes(M, N, K) : 0;
    const size_t fused = small > cols ? small : cols;
    return fused > tall ? fused : tall;
}

template <int BITS, int MT>
static void launch_gemm(hipStream_t stream, const GemmPlan& p, const void* x, const int32_t* qweight,
                        const int32_t* qzeros, const void* scales, void* out, void* workspace, int M, int N,
                        int K, int group_size) {
    // the arrival counters at the head of the workspace belong to the small-M kernel
    float* partial = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + kTileCounterBytes);
    hipLaunchKernelGGL((gptq_gemm_kernel<BITS, MT>), dim3(p.col_tiles, p.split_k, p.m_blocks), dim3(256), 0,
                       stream, (const half_t*)x, (const uint32_t*)qweight, (const uint32_t*)qzeros,
                       (const half_t*)scales, (half_t*)out, partial, M, N, K, group_size / 32,
                       p.steps_total, p.steps_per_block, p.split_k);
    if (p.split_k > 1) launch_splitk_finalize(stream, partial, out, M, N, p.split_k, kEpilogueNone, SmallFuse{});
}


template <int BITS, int MT>
static void launch_gemm_small(hipStream_t stream, const GemmPlan& p, const void* x, const int32_t* qweight,
                              const int32_t* qzeros, const void* scales, void* out, void* workspace, int M,
                              int N, int K, int group_size, int epilogue, const SmallFuse& fuse) {
    // workspace: [tile counters, zero between launches][fp32 partials]
    // in-kernel reduction by the last workgroup of a tile pays for few rows only
    // (a tile whose two K shares sit in one workgroup and that is not split further has one contributor: its
    // epilogue runs in the launch at any row count, small_two_shares)
    // (a plain product of five to eight rows whose tiles have more than sixteen contributors goes to the second
    // stage all the same: one workgroup reading that many partial tiles is slower than a launch that spreads
    // them over the chip -- 14336 x 4096 at 5-8 rows, 28 contributors, 17.0-17.3 -> 14.2-14.9 us; with sixteen
    // contributors, 28672 x 8192, 26.3-27.5 us in the kernel against 28.3-30.2)
    const bool many_contributors = epilogue == kEpilogueNone && fuse.ssq_in == nullptr && p.stream_units == 0 &&
                                   M > 4 && p.split_k > 16;
    unsigned* counters = ((M <= kFusedReduceMaxM || (p.k_ways == 2 && p.split_k == 1)) && p.col_tiles <= kMaxTileCounters &&
                          !many_contributors)
                             ? reinterpret_cast<unsigned*>(workspace)
                             : nullptr;
    float* partial = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + kTileCounterBytes);
    const dim3 grid = p.stream_units ? dim3(p.blocks) : dim3(p.col_tiles, p.split_k, p.m_blocks);
    const bool norm = fuse.ssq_in != nullptr;
#define MH_LAUNCH_SMALL_K(SPG, NORM, STREAM, KW)                                                                  \
    hipLaunchKernelGGL((gptq_gemm_small_kernel<BITS, MT, SPG, NORM, STREAM, KW>), grid, dim3(256 * KW), 0, stream, \
                       (const half_t*)x, (const uint32_t*)qweight, (const uint32_t*)qzeros, (const half_t*)scales, \
                       (half_t*)out, partial, counters, M, N, K, p.steps_total, p.steps_per_block / kSmallDepth,  \
                       p.split_k, p.stream_units, epilogue, fuse)
#define MH_LAUNCH_SMALL_N(SPG, NORM, STREAM)                     \
    do {                                                         \
        if constexpr (MT <= 2 && !(STREAM) && SPG >= 2) {        \
            if (p.k_ways == 2) {                                 \
                MH_LAUNCH_SMALL_K(SPG, NORM, false, 2);          \
                break;                                           \
            }                                                    \
        }                                                        \
        MH_LAUNCH_SMALL_K(SPG, NORM, STREAM, 1);                 \
    } while (0)
#define MH_LAUNCH_SMALL(SPG)                                     \
    do {                                                         \
        if constexpr (MT <= 2) {                                 \
            if (norm) {                                          \
                MH_LAUNCH_SMALL_N(SPG, true, false);             \
                break;                                           \
            }                                                    \
            if (MT == 1 && p.stream_units != 0) {                \
                MH_LAUNCH_SMALL_N(SPG, false, (MT == 1));        \
                break;                                           \
            }                                                    \
        }                                                        \
        MH_LAUNCH_SMALL_N(SPG, false, false);                    \
    } while (0)
    switch (group_size / 32) {
        case 1: MH_LAUNCH_SMALL(1); break;
        case 2: MH_LAUNCH_SMALL(2); break;
        case 4: MH_LAUNCH_SMALL(4); break;
        default: MH_LAUNCH_SMALL(8); break;
    }
#undef MH_LAUNCH_SMALL
#undef MH_LAUNCH_SMALL_N
#undef MH_LAUNCH_SMALL_K
    if (counters == nullptr && (p.split_k > 1 || epilogue != kEpilogueNone))
        launch_splitk_finalize(stream, partial, out, M, N, p.split_k, epilogue, fuse);
}

template <int BITS>
static void launch_gemm_mt(hipStream_t stream, const GemmPlan& p, const void* x, const int32_t* qweight,
                           const int32_t* qzeros, const void* scales, void* out, void* workspace, int M,
                           int N, int K, int group_size, int epilogue, const SmallFuse& fuse) {
    if (use_small(M, group_size)) {
        if (p.mt == 1)
            launch_gemm_small<BITS, 1>(stream, p, x, qweight, qzeros, scales, out, workspace, M, N, K, group_size,
                                       epilogue, fuse);
        else
            launch_gemm_small<BITS, 2>(stream, p, x, qweight, qzeros, scales, out, workspace, M, N, K, group_size,
                                       epilogue, fuse);
        return;
    }
    switch (p.mt) {
        case 1: launch_gemm<BITS, 1>(stream, p, x, qweight, qzeros, scales, out, workspace, M, N, K, group_size); break;
        case 2: launch_gemm<BITS, 2>(stream, p, x, qweight, qzeros, scales, out, workspace, M, N, K, group_size); break;
        case 4: launch_gemm<BITS, 4>(stream, p, x, qweight, qzeros, scales, out, workspace, M, N, K, group_size); break;
        default: launch_gemm<BITS, 8>(stream, p, x, qweight, qzeros, scales, out, workspace, M, N, K, group_size); break;
    }
}

int gptq_gemm_launch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                     const void* scales, void* out, int M, int N, int K, int group_size, int bits,
                     void* workspace, size_t workspace_bytes, int epilogue, const SmallFuse& fuse) {
    // the MFMA kernels address the packed weights with 32-bit buffer offsets
    if (!packed_weights_addressable(N, K, bits))
        return fail(MH_ERR_INVALID, "gptq gemm: packed weights of 2 GiB or more are not supported by the MFMA kernels "
                    "(mh_gptq_matmul serves them with the per-element kernel)");
    // more than 64 rows: blocks of 128 rows, a packed word dequantised once per block
    if (fuse.ssq_in == nullptr && gemm_tall_preferred(M, N, K, group_size, bits, epilogue))
        return gptq_gemm_tall_launch(stream, x, qweight, qzeros, scales, out, M, N, K, group_size, workspace,
                                     workspace_bytes, fuse.bias, kEpilogueNone);
    if (fuse.ssq_in == nullptr && epilogue == kEpilogueSiluPairs && gemm_tall_silu_pairs_supported(M, N, K, group_size, bits))
        return gptq_gemm_tall_launch(stream, x, qweight, qzeros, scales, out, M, N, K, group_size, workspace,
                                     workspace_bytes, nullptr, kEpilogueSiluPairs);
    // many rows: the kernel that dequantises a weight tile once for 128 rows
    if (fuse.ssq_in == nullptr && gemm_wide_preferred(M, N, K, group_size, bits, epilogue))
        return gptq_gemm_wide_launch(stream, x, qweight, qzeros, scales, out, M, N, K, group_size, workspace,
                                     workspace_bytes, fuse.bias);
    // a narrow output goes to the kernel whose workgroups own their columns over all of K
    if (gemm_cols_preferred(M, N, K, group_size, bits, epilogue))
        return gptq_gemm_cols_launch(stream, x, qweight, qzeros, scales, out, M, N, K, group_size, bits, epilogue, fuse,
                                     workspace, workspace_bytes);
    if (row_blocked(M, group_size)) {
        // Above kSmallMaxM rows the small-M kernel takes blocks of 64 rows (four 16-row
        // tiles per workgroup) side by side in one launch: the packed weights are read
        // once per block of rows, the second reader mostly from a cache.  Measured
        // 2-5x faster at M = 64..128 than the staged kernel, whose few large
        // workgroups leave most CUs idle.
        if (epilogue != kEpilogueNone || fuse.ssq_in != nullptr)
            return fail(MH_ERR_INVALID, "gptq gemm: epilogues and norm fusion need M <= %d", kSmallMaxM);
        const size_t need = gemm_workspace_bytes(M, N, K, group_size, bits);
        if (need != 0 && (workspace == nullptr || workspace_bytes < need))
            return fail(MH_ERR_WORKSPACE, "mh_gptq_gemm: workspace of %zu bytes required, got %zu", need,
                        workspace ? workspace_bytes : (size_t)0);
        if (need != 0 && (uintptr_t)workspace % 256 != 0)
            return fail(MH_ERR_WORKSPACE, "mh_gptq_gemm: workspace must be 256-byte aligned");
        // one launch: blockIdx.z walks the blocks of kSmallBlockM rows
        const GemmPlan p = plan_gemm_small(kSmallBlockM, N, K, false, (M + kSmallBlockM - 1) / kSmallBlockM);
        if (bits == 4)
            launch_gemm_small<4, 4>(stream, p, x, qweight, qzeros, scales, out, workspace, M, N, K, group_size,
                                    kEpilogueNone, fuse);
        else
            launch_gemm_small<8, 4>(stream, p, x, qweight, qzeros, scales, out, workspace, M, N, K, group_size,
                                    kEpilogueNone, fuse);
        MH_CHECK_LAUNCH();
        return MH_OK;
    }
    const GemmPlan p = plan_gemm(M, N, K, group_size, epilogue == kEpilogueNone && fuse.ssq_in == nullptr, bits);
    if ((fuse.ssq_in != nullptr || epilogue == kEpilogueResidual || epilogue == kEpilogueRopeAppend) &&
        !gemm_norm_fusion_supported(M, N, K, group_size, bits, epilogue))
        return fail(MH_ERR_INVALID, "gptq gemm: RMSNorm / RoPE fusion needs M <= %d, a group of 32..256 and N %% 256 == 0 "
                    "(N %% 1024 == 0 above %d rows)", kSmallMaxM, kFusedReduceMaxM);
    const size_t need = gemm_workspace_bytes(M, N, K, group_size, bits);
    if (epilogue != kEpilogueNone && !gemm_silu_pairs_supported(M, N, K, group_size, bits))
        return fail(MH_ERR_INVALID, "gptq gemm: the SiLU-pair epilogue needs M <= %d, N %% 256 == 0 and a group of 32..256",
                    kSmallMaxM);
    if (p.split_k > 1 || epilogue != kEpilogueNone) {
        if (workspace == nullptr || workspace_bytes < need)
            return fail(MH_ERR_WORKSPACE, "mh_gptq_gemm: workspace of %zu bytes required, got %zu", need,
                        workspace ? workspace_bytes : (size_t)0);
        if ((uintptr_t)workspace % 256 != 0)
            return fail(MH_ERR_WORKSPACE, "mh_gptq_gemm: workspace must be 256-byte aligned");
    }
    if (bits == 4)
        launch_gemm_mt<4>(stream, p, x, qweight, qzeros, scales, out, workspace, M, N, K, group_size, epilogue, fuse);
    else
        launch_gemm_mt<8>(stream, p, x, qweight, qzeros, scales, out, workspace, M, N, K, group_size, epilogue, fuse);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

int gemv_gemm_crossover() {
    // measured on MI355X: the MFMA kernel is at least as fast from M = 1 on
    static const int m = env_int_gemm("MH_GEMV_MAX_M", 0);
    return m < MH_GPTQ_GEMV_MAX_M ? m : MH_GPTQ_GEMV_MAX_M;
}

}  // namespace mh
