// GPTQ w4a16 / w8a16 product for a few rows where the output is narrow: one
// workgroup owns 32 output columns over all of K.
//
// The small-M kernel (gptq_gemm.hip) cuts a narrow output into 256-column tiles
// and needs 11-16 K splits per tile to fill the GPU; the partial sums then cross
// workgroups (agent-scope stores, an arrival counter, a reload by the last
// workgroup), three dependent memory round trips of about a microsecond each at
// the end of a 10 us kernel.  Here K is split over the eight waves of the one
// workgroup that owns the columns and the partial sums meet in LDS.
//
// A wave walks its own contiguous K range, so it shares nothing with the other
// waves until the end and the K loop has no barrier.  Per step of 32 k a lane
// (column pair nl = lane % 16, k chunk kq = lane / 16) loads 8 bytes: the packed
// words of its two columns, which are the B operands of two
// v_mfma_f32_16x16x32_f16.  Everything a step needs is requested 8 steps ahead
// and in the order of use (activations of a 256-k stage, scale/zero words of a
// group, packed weights), so each s_waitcnt vmcnt(n) leaves the 8 steps behind it
// in flight: 4 KiB per wave, 32 KiB per CU.  More in flight measured slower (16
// steps: 8192x8192 in 11.4 us instead of 9.8; a 16-byte-per-lane variant with
// 128 KiB per CU: 14.7 us), and beyond about 34 loads in flight per wave the
// compiler's vmcnt bookkeeping falls back to draining the queue at the top of the
// loop.  Activations go through a wave-private LDS area (re-ordered to the pair
// order of dequant_word on the way); LDS instructions of one wave execute in
// order, so the area needs neither a second buffer nor a barrier.
//
// Measured against the small-M kernel (M = 1, us): 8192x8192 9.8 / 15.3,
// 4096x4096 5.8 / 9.1, 16384x8192 15.7 / 22.3, 28672x8192 24.5 / 26.2 (at 8 rows
// 29.8 / 28.2).  With more 32-column tiles than CUs it loses when the extra tiles
// make a second round (10240 columns: 15.9 / 15.0) and gains a little when they
// are cut along K instead (14.1 / 15.0, see the kernel); with half the CUs idle
// on a long K (14336x4096: 16.6 / 14.8) it loses.  gemm_cols_preferred decides.
// 8-bit weights (two packed rows per lane and step): 8192x8192 14.6 / 18.1,
// 4096x4096 8.4 / 9.9.
// A wide output (8192x57344, 1792 tiles) stays with the small-M kernel (48 us): one
// tile per workgroup here takes 60 us, and a variant whose workgroups walked seven
// tiles as one stream (activations parked in LDS once, the ring running across tile
// borders, one barrier per tile) took 53 us with adjacent tiles per workgroup and
// 60 us with tiles interleaved across workgroups.
#include "gptq_common.h"

namespace mh {

#pragma clang fp contract(off)

constexpr int kColsTile = 32;   // columns per workgroup
constexpr int kColsWaves = 8;     // K ranges per workgroup (16 measured slower: 8192x8192 10.5 against 10.0 us, 28672x8192 25.0 against 24.5)
constexpr int kColsCutWaves = 4;  // on the cut plan, where a CU holds a whole tile and a part: 8192x10240 12.3 against 14.3 us with 8
                                  // (with the norm prologue, RoPE and cache append of the decode loop: 12.1 against 13.6)
constexpr int kColsStage = 8;   // steps per activation stage
constexpr int kColsRing = 8;    // steps in flight per wave
constexpr int kColsParts = 4;  // K ranges of a tile that is cut, when there are more tiles than CUs

template <int BITS, int SPG, int MROWS, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gptq_gemm_cols_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ qweight, const uint32_t* __restrict__ qzeros,
    const half_t* __restrict__ scales, half_t* out, float* partial, unsigned* counters, int M, int N, int K,
    int steps_total, int steps_per_wave, int full_tiles, int parts, int part_steps_per_wave, int epilogue,
    SmallFuse fuse) {
    constexpr int P = Packing<BITS>::kPerWord;
    constexpr int PAIRS = Packing<BITS>::kPairs;
    constexpr uint32_t MASK = Packing<BITS>::kMask;
    constexpr int R = kColsRing;
    constexpr int ROWS_PER_STEP = 32 / P;
    constexpr int LOADS = ROWS_PER_STEP / 4;
    constexpr int CS = R / SPG;                          // scale/zero slots
    constexpr int MT = MROWS > 16 ? 2 : 1;               // 16-row tiles of the activations
    constexpr int STAGE = MROWS > 16 ? 4 : kColsStage;   // steps per activation stage (LDS: rows x stage per wave)
    constexpr int CH = STAGE * 4;                        // 16-byte chunks per row and stage
    constexpr int XS = R / STAGE;                        // activation stage slots
    constexpr int XP = MROWS * CH > 64 ? MROWS * CH / 64 : 1;  // 16-byte chunks per lane and stage
    constexpr int RS = CH + 1;                           // padded row stride of the staging area
    constexpr int SSQ_ROWS = (MROWS * 32 + WAVES * 64 - 1) / (WAVES * 64);  // rows per 32 threads, norm prologue
    static_assert(R % STAGE == 0 && R % SPG == 0 && kColsStage % STAGE == 0, "slots must divide the ring");
    static_assert(MROWS * (kColsTile / 2) <= WAVES * 64, "one thread per row and column pair");

    __shared__ uint4 xs[WAVES][MROWS * RS];
    __shared__ float red[WAVES][MROWS][kColsTile];
    __shared__ float inv_rms_s[MROWS];
    __shared__ int is_last;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nl = lane & 15, kq = lane >> 4;
    // Workgroups 0 .. full_tiles - 1 own a tile over all of K.  Where there are a few
    // more tiles than CUs, the remaining tiles are cut into `parts` K ranges, one
    // workgroup each, so that every CU gets one whole tile and at most one part; the
    // parts' sums cross workgroups (see the results section), which ends long
    // before the whole tiles are through.
    int tile = blockIdx.x, part = 0, nparts = 1;
    if (tile >= full_tiles) {
        const int s = tile - full_tiles;
        tile = full_tiles + s / parts;
        part = s % parts;
        nparts = parts;
        steps_per_wave = part_steps_per_wave;
    }
    const int col0 = tile * kColsTile + nl * 2;

    const int begin = (part * WAVES + wave) * steps_per_wave;
    const int end = min(begin + steps_per_wave, steps_total);
    const int last_step = steps_total - 1;
    const int last_stage_step = (last_step / STAGE) * STAGE;
    const int ring_last = max(min(end, steps_total) - 1, 0);

    // ---- packed weights
    uint2_t qb[R][LOADS];
    uint32_t lane_off[LOADS];
#pragma unroll
    for (int j = 0; j < LOADS; ++j) lane_off[j] = (uint32_t)((kq * LOADS + j) * N + col0) * 4u;
    // buffer loads: scalar offset of the step + the lane's fixed 32-bit offset, no
    // vector address arithmetic; streaming hint, agent scope
    const __amdgpu_buffer_rsrc_t q_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(qweight), 0, (int)((size_t)(K / P) * N * 4), kBufferRsrcFlags);
    auto load_q = [&](int step, uint2_t* dst) {
        // past the end of the wave's range: re-read its last step (a cache hit; running on
        // into the next wave's range measured 10 % more HBM traffic), its activations are zero
        const int s = min(step, ring_last);
        const int soff = s * ROWS_PER_STEP * N * 4;
#pragma unroll
        for (int j = 0; j < LOADS; ++j)
            dst[j] = __builtin_bit_cast(
                uint2_t, __builtin_amdgcn_raw_buffer_load_b64(q_rsrc, (int)lane_off[j], soff, kBufferStreamAgent));
    };

    // ---- scales and zero points of a group: one word each for the lane's two columns
    uint32_t cs_scale[CS], cs_zero[CS];
    const int zsub = col0 % P;
    auto load_c = [&](int step, int slot) {
        const int g = min(step, last_step) / SPG;
        cs_scale[slot] = *reinterpret_cast<const uint32_t*>(scales + (size_t)g * N + col0);
        cs_zero[slot] = qzeros[(size_t)g * (N / P) + col0 / P];
    };

    // ---- activations of a stage: lane -> (row, 16-byte chunk) of its wave's stage
    uint4 xr[XS][XP];
    int x_row[XP], x_chunk[XP];
#pragma unroll
    for (int u = 0; u < XP; ++u) {
        const int item = u * 64 + lane;
        x_row[u] = min(item / CH, M - 1);
        x_chunk[u] = item % CH;
    }
    auto load_x = [&](int step, int slot) {
        const int s = min(step, last_stage_step);
#pragma unroll
        for (int u = 0; u < XP; ++u)
            xr[slot][u] = *reinterpret_cast<const uint4*>(x + (size_t)x_row[u] * K + (size_t)s * 32 + x_chunk[u] * 8);
    };
    auto store_x = [&](int step, int slot) {
#pragma unroll
        for (int u = 0; u < XP; ++u) {
            const uint32_t in[4] = {xr[slot][u].x, xr[slot][u].y, xr[slot][u].z, xr[slot][u].w};
            uint32_t o[4];
            if constexpr (BITS == 4) {
                pair_activations<4>(in, o);
            } else {
                pair_activations<8>(in, o);
                pair_activations<8>(in + 2, o + 2);
            }
            const bool live = step + x_chunk[u] / 4 < end;  // steps of another wave or past K add nothing
            if (u * 64 + lane < MROWS * CH)
                xs[wave][(u * 64 + lane) / CH * RS + x_chunk[u]] =
                    live ? make_uint4(o[0], o[1], o[2], o[3]) : make_uint4(0, 0, 0, 0);
        }
    };

    // the producer's sums of squares (norm prologue) are requested ahead of everything
    // else, so that waiting for them below leaves the ring in flight
    const int ssq_p0 = tid & 31;
    int ssq_row[SSQ_ROWS];
    bool ssq_mine[SSQ_ROWS];
    const float* ssq_pieces[SSQ_ROWS];
    SsqLane ssq_part[SSQ_ROWS] = {};
#pragma unroll
    for (int j = 0; j < SSQ_ROWS; ++j) {
        ssq_row[j] = (tid >> 5) + j * (WAVES * 2);
        ssq_mine[j] = fuse.ssq_in != nullptr && ssq_row[j] < M;
        ssq_pieces[j] = fuse.ssq_in + (size_t)(ssq_mine[j] ? ssq_row[j] : 0) * fuse.ssq_tiles;
        if (ssq_mine[j]) ssq_part[j] = ssq_lane_load(ssq_pieces[j], fuse.ssq_tiles, ssq_p0);
    }

    // Operands of the epilogue that do not depend on the product are requested here as
    // well (the row's position now, what hangs on it after the ring): at the end of
    // the kernel each would be a dependent round trip on the critical path.
    const bool ep_worker = tid < M * (kColsTile / 2);  // one thread per (row, column pair) of the tile
    const int ep_m = tid / (kColsTile / 2), ep_col = tile * kColsTile + tid % (kColsTile / 2) * 2;
    int ep_pos = 0;
    if (epilogue == kEpilogueRopeAppend && ep_worker) ep_pos = fuse.positions[ep_m];

    // requests in the order of use
#pragma unroll
    for (int d = 0; d < R; ++d) {
        if (d % STAGE == 0) load_x(begin + d, d / STAGE);
        if (d % SPG == 0) load_c(begin + d, d / SPG);
        load_q(begin + d, qb[d]);
    }

    half2_t ep_h = {(half_t)0.f, (half_t)0.f}, ep_w = {(half_t)0.f, (half_t)0.f};
    float ep_cos = 0.f, ep_sin = 0.f;
    if (ep_worker) {
        if (epilogue == kEpilogueResidual) {
            ep_h = *reinterpret_cast<const half2_t*>(out + (size_t)ep_m * N + ep_col);
            if (fuse.xw_out) ep_w = *reinterpret_cast<const half2_t*>(fuse.next_norm_w + ep_col);
        } else if (epilogue == kEpilogueRopeAppend) {
            ep_pos = min(max(ep_pos, 0), fuse.max_seq - 1);
            ep_cos = fuse.rope_cos[(size_t)ep_pos * 64 + ep_col % 128 / 2];
            ep_sin = fuse.rope_sin[(size_t)ep_pos * 64 + ep_col % 128 / 2];
        }
    }

    if (fuse.ssq_in != nullptr) {
        // 1 / rms of the rows from the producer's sums of squares (see SmallFuse): 32
        // lanes per row, folded by shuffles in a fixed order; read after the K loop
#pragma unroll
        for (int j = 0; j < SSQ_ROWS; ++j) {
            float ss = 0.f;
            if (ssq_mine[j]) ss = ssq_lane_sum(ssq_part[j], ssq_pieces[j], fuse.ssq_tiles, ssq_p0);
#pragma unroll
            for (int off = 1; off < 32; off <<= 1) ss += __shfl_xor(ss, off);
            if (ssq_p0 == 0 && ssq_row[j] < MROWS) inv_rms_s[ssq_row[j]] = 1.f / sqrtf(ss / (float)K + fuse.eps);
        }
    }

    DequantRegs regs;
    regs.init(BITS);
    float4_t acc[MT][2];
    int a_row[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        acc[mt][0] = acc[mt][1] = float4_t{0.f, 0.f, 0.f, 0.f};
        a_row[mt] = min(mt * 16 + nl, M - 1);
    }
    ColumnConst cc[2];

    for (int base = 0; base < steps_per_wave; base += R) {
        // The two waves of a SIMD are not served alike: the older one wins every arbitration, and
        // without this the first four waves of a workgroup leave the loop 5.3 us before the last
        // four on 28672 x 8192 (1.6 us on 8192 x 8192), which then stream alone.  The priority of
        // a wave falls with its progress through its K range, so the one behind is served first.
        // (Not on the cut plan, where a CU holds two workgroups of unequal ranges: 0.4 us slower there.)
        if (parts == 1) set_priority_by_progress(base, steps_per_wave);
#pragma unroll
        for (int d = 0; d < R; ++d) {
            const int step = begin + base + d;
            if (d % STAGE == 0) {
                store_x(step, d / STAGE);
                load_x(step + R, d / STAGE);
            }
            if (d % SPG == 0) {
                const uint32_t sw = cs_scale[d / SPG], zw = cs_zero[d / SPG];
                cc[0] = column_const_from_bits(sw & 0xFFFFu, (zw >> (zsub * BITS)) & MASK);
                cc[1] = column_const_from_bits(sw >> 16, (zw >> ((zsub + 1) * BITS)) & MASK);
                load_c(step + R, d / SPG);
            }
            half8_t b[2];
            uint2_t* q = qb[d];
            const uint32_t qa[2] = {q[0].x, q[0].y};
            const uint32_t qc[2] = {q[LOADS - 1].x, q[LOADS - 1].y};
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                half2_t w[4];
                dequant_word<BITS>(qa[t], cc[t], regs, w);
                if constexpr (BITS == 8) dequant_word<BITS>(qc[t], cc[t], regs, w + PAIRS);
                const uint4_t packed = {as_u32(w[0]), as_u32(w[1]), as_u32(w[2]), as_u32(w[3])};
                b[t] = __builtin_bit_cast(half8_t, packed);
            }
            load_q(step + R, q);
            __builtin_amdgcn_sched_barrier(0);  // keeps the reload at this place of the body
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const half8_t a = __builtin_bit_cast(half8_t, xs[wave][a_row[mt] * RS + (d % STAGE) * 4 + kq]);
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b[t], acc[mt][t], 0, 0, 0);
            }
        }
    }

    // ---- the eight partial sums of a column meet in LDS, in wave order
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = mt * 16 + kq * 4 + r;
            if (m < M) *reinterpret_cast<float2*>(&red[wave][m][nl * 2]) = make_float2(acc[mt][0][r], acc[mt][1][r]);
        }
    __syncthreads();
    const bool worker = tid < M * (kColsTile / 2);  // one thread per (row, column pair)
    const int m = tid / (kColsTile / 2), c = tid % (kColsTile / 2) * 2;
    const int col = tile * kColsTile + c;
    float2 sum = make_float2(0.f, 0.f);
    if (worker) {
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float2 v = *reinterpret_cast<const float2*>(&red[w][m][c]);
            sum.x += v.x;
            sum.y += v.y;
        }
    }
    if (nparts > 1) {
        // a tile cut along K: publish, count in, and the workgroup that arrives last
        // adds the parts in part order (common.h:arrive_and_check_last)
        const size_t plane = (size_t)M * N;
        if (worker) {
            float* dst = partial + (size_t)part * plane + (size_t)m * N + col;
            store_agent(dst, sum.x);
            store_agent(dst + 1, sum.y);
        }
        if (!arrive_and_check_last(&counters[tile], (unsigned)nparts, &is_last)) return;
        if (worker) {
            // the parts are requested together and added in part order (nparts is kColsParts here)
            float2 v[kColsParts];
#pragma unroll
            for (int p = 0; p < kColsParts; ++p) {
                const float* src = partial + (size_t)min(p, nparts - 1) * plane + (size_t)m * N + col;
                v[p] = make_float2(load_agent(src), load_agent(src + 1));
            }
            sum = make_float2(0.f, 0.f);
#pragma unroll
            for (int p = 0; p < kColsParts; ++p)
                if (p < nparts) {
                    sum.x += v[p].x;
                    sum.y += v[p].y;
                }
        }
    }
    if (!worker) return;
    if (fuse.ssq_in != nullptr) {
        const float inv = inv_rms_s[m];
        sum.x *= inv;
        sum.y *= inv;
    }
    half2_t y = {(half_t)sum.x, (half_t)sum.y};
    if (fuse.bias) y = y + *reinterpret_cast<const half2_t*>(fuse.bias + col);  // before any epilogue
    half2_t* op = reinterpret_cast<half2_t*>(out + (size_t)m * N + col);
    if (epilogue == kEpilogueResidual) {
        // out is the residual stream: h += y in fp16, h * next_norm_w for the consumer,
        // and the sum of squares of the tile's 32 new values (the row's 16 threads
        // are adjacent lanes of one wave)
        const half2_t h = ep_h + y;  // ep_h: this thread's two elements of the stream, read at the start
        *op = h;
        if (fuse.xw_out) *reinterpret_cast<half2_t*>(fuse.xw_out + (size_t)m * N + col) = norm_weighted(h, ep_w, fuse.xw_clamped);
        float ss = (float)h[0] * (float)h[0] + (float)h[1] * (float)h[1];
#pragma unroll
        for (int off = 1; off < kColsTile / 2; off <<= 1) ss += __shfl_xor(ss, off);
        if (c == 0) fuse.ssq_out[(size_t)m * (N / kColsTile) + tile] = ss;
        return;
    }
    if (epilogue == kEpilogueRopeAppend) {
        // the two columns are one interleaved pair of a head of 128 dims (gptq_common.h)
        const int head = col / 128, d = col % 128;
        const int pos = ep_pos;  // clamped to the cache at the start
        if (head >= fuse.q_heads + fuse.kv_heads) {  // value head: copied, cache is tiled
            half_t* dst = fuse.vt_cache + ((size_t)m * fuse.kv_heads + (head - fuse.q_heads - fuse.kv_heads)) * 128 * fuse.max_seq +
                          vt_offset(d, pos);
            dst[0] = y[0];
            dst[kVTile] = y[1];
            return;
        }
        const float cs = ep_cos, sn = ep_sin;
        const float re = (float)y[0], im = (float)y[1];
        const half2_t o = {(half_t)(re * cs - im * sn), (half_t)(im * cs + re * sn)};
        half_t* dst = head < fuse.q_heads
                          ? fuse.q_out + ((size_t)m * fuse.q_heads + head) * 128 + d
                          : fuse.k_cache + (((size_t)m * fuse.kv_heads + (head - fuse.q_heads)) * fuse.max_seq + pos) * 128 + d;
        *reinterpret_cast<half2_t*>(dst) = o;
        return;
    }
    *op = y;
}

bool gemm_cols_supported(int M, int N, int K, int group_size, int bits, int epilogue) {
    static const char* off = getenv("MH_GEMM_NO_COLS");
    if (off && *off && atoi(off)) return false;
    if ((bits != 4 && bits != 8) || M < 1 || M > 32) return false;
    if (group_size != 32 && group_size != 64 && group_size != 128 && group_size != 256) return false;
    if (N % kColsTile != 0 || K % (32 * kColsStage) != 0) return false;
    return epilogue == kEpilogueNone || epilogue == kEpilogueResidual || epilogue == kEpilogueRopeAppend;
}

// Tiles beyond one per CU are cut into kColsParts K ranges, which must not outnumber the CUs.
static int cols_waves(int M, bool cut) { return cut && M <= 8 ? kColsCutWaves : kColsWaves; }
static bool cols_cut_plan(int M, int tiles, int K, int cus) {
    return tiles > cus && (tiles - cus) * kColsParts <= cus && tiles - cus < kMaxTileCounters &&
           K % (32 * kColsStage * cols_waves(M, true) * kColsParts) == 0;
}
// The cut plan is taken up to eight rows (8192x10240 against the small-M kernel: 13.4 /
// 15.8 us at 3 rows, 14.5 / 16.7 at 8; with eight waves per workgroup it had shown no
// gain at 8 rows).
static bool cols_use_cut(int M, int tiles, int K, int cus) {
    static const char* nocut = getenv("MH_GEMM_COLS_NO_CUT");
    // above 8 rows (eight waves per workgroup) the small-M kernel is faster: 8192x10240 at
    // 12 / 16 / 32 rows 21.0 / 21.7 / 28.8 us against 18.7 / 19.4 / 25.5
    return M <= 8 && cols_cut_plan(M, tiles, K, cus) && !(nocut && *nocut && atoi(nocut));
}

// Where it measured faster than the small-M kernel: every CU gets at most one
// 32-column tile (plus at most one K range of a cut tile), and either the tiles
// cover more than half the CUs or K is short enough for the kernel to be bound by
// its dependent round trips rather than by the CUs left idle.
bool gemm_cols_preferred(int M, int N, int K, int group_size, int bits, int epilogue) {
    if (!gemm_cols_supported(M, N, K, group_size, bits, epilogue)) return false;
    static const char* force = getenv("MH_GEMM_COLS_FORCE");
    if (force && *force && atoi(force)) return true;
    const int tiles = N / kColsTile, cus = compute_units();
    // the thresholds were measured on 4-bit weights; 8-bit rows carry twice the bytes per k
    const long kb = (long)K * bits / 4;
    // measured at 8192x10240 (320 tiles on 256 CUs): 12.7 against 15.0 us at M = 1
    if (cols_use_cut(M, tiles, K, cus)) return kb <= 8192;
    // 28672x8192 against the small-M kernel: 26.5 / 27.5 us at M = 3, 27.0 / 27.6 at 4, equal at 6, 30.2 / 29.2 at 8
    return tiles <= cus && (kb <= 8192 || 2 * tiles > cus) && (kb <= 16384 || M <= 4);
}

// Bytes of workspace a launch of this kernel needs for the shape (0: none).
size_t gemm_cols_workspace_bytes(int M, int N, int K) {
    return cols_cut_plan(M, N / kColsTile, K, compute_units()) ? kTileCounterBytes + (size_t)kColsParts * M * N * sizeof(float)
                                                            : 0;
}

int gptq_gemm_cols_launch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                          const void* scales, void* out, int M, int N, int K, int group_size, int bits, int epilogue,
                          const SmallFuse& fuse, void* workspace, size_t workspace_bytes) {
    if (!gemm_cols_supported(M, N, K, group_size, bits, epilogue))
        return fail(MH_ERR_INVALID, "gptq column-owner kernel: unsupported shape or fusion");
    const int steps_total = K / 32;
    const int tiles = N / kColsTile, cus = compute_units();
    const bool cut = cols_use_cut(M, tiles, K, cus);
    const int waves = cols_waves(M, cut);
    int spw = (steps_total + waves - 1) / waves;
    spw = (spw + kColsStage - 1) / kColsStage * kColsStage;  // whole stages, hence whole groups
    int full_tiles = tiles, parts = 1, part_spw = spw;
    float* partial = nullptr;
    unsigned* counters = nullptr;
    if (cut) {
        const size_t need = gemm_cols_workspace_bytes(M, N, K);
        if (workspace == nullptr || workspace_bytes < need)
            return fail(MH_ERR_WORKSPACE, "mh_gptq_gemm: workspace of %zu bytes required, got %zu", need,
                        workspace ? workspace_bytes : (size_t)0);
        full_tiles = cus;
        parts = kColsParts;
        part_spw = steps_total / (waves * kColsParts);
        counters = reinterpret_cast<unsigned*>(workspace);
        partial = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + kTileCounterBytes);
    }
    const dim3 grid(full_tiles + (tiles - full_tiles) * parts);
#define MH_LAUNCH_COLS_W(BITS, SPG, MROWS, WAVES)                                                                  \
    hipLaunchKernelGGL((gptq_gemm_cols_kernel<BITS, SPG, MROWS, WAVES>), grid, dim3(WAVES * 64), 0, stream,        \
                       (const half_t*)x, (const uint32_t*)qweight, (const uint32_t*)qzeros, (const half_t*)scales, \
                       (half_t*)out, partial, counters, M, N, K, steps_total, spw, full_tiles, parts, part_spw,    \
                       epilogue, fuse)
// the cut plan runs with kColsCutWaves waves per workgroup up to eight rows (above, a
// workgroup of eight waves is what gives every row and column pair its thread)
#define MH_LAUNCH_COLS_B(BITS, SPG, MROWS)                               \
    do {                                                                 \
        if constexpr (MROWS <= 8) {                                      \
            if (cut) {                                                   \
                MH_LAUNCH_COLS_W(BITS, SPG, MROWS, kColsCutWaves);       \
                break;                                                   \
            }                                                            \
        }                                                                \
        MH_LAUNCH_COLS_W(BITS, SPG, MROWS, kColsWaves);                  \
    } while (0)
#define MH_LAUNCH_COLS_S(BITS, MROWS)                        \
    switch (group_size / 32) {                               \
        case 1: MH_LAUNCH_COLS_B(BITS, 1, MROWS); break;     \
        case 2: MH_LAUNCH_COLS_B(BITS, 2, MROWS); break;     \
        case 4: MH_LAUNCH_COLS_B(BITS, 4, MROWS); break;     \
        default: MH_LAUNCH_COLS_B(BITS, 8, MROWS); break;    \
    }
#define MH_LAUNCH_COLS(MROWS)           \
    do {                                \
        if (bits == 4) {                \
            MH_LAUNCH_COLS_S(4, MROWS)  \
        } else {                        \
            MH_LAUNCH_COLS_S(8, MROWS)  \
        }                               \
    } while (0)
    if (M == 1)
        MH_LAUNCH_COLS(1);
    else if (M == 2)
        MH_LAUNCH_COLS(2);
    else if (M <= 4)
        MH_LAUNCH_COLS(4);
    else if (M <= 8)
        MH_LAUNCH_COLS(8);
    else if (M <= 16)
        MH_LAUNCH_COLS(16);
    else
        MH_LAUNCH_COLS(32);
#undef MH_LAUNCH_COLS_W
#undef MH_LAUNCH_COLS_B
#undef MH_LAUNCH_COLS_S
#undef MH_LAUNCH_COLS
    MH_CHECK_LAUNCH();
    return MH_OK;
}

}  // namespace mh
