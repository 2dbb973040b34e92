// W8A8 int8 GEMM on CDNA4 int8 MFMA (v_mfma_i32_32x32x32_i8) with exact int32
// accumulation and a per-token x per-channel scale epilogue.
//
// The reference has no int8 x int8 product; the operand orientation is the one
// of its dense MatrixMultiply, C[m, n] = sum_k A[m, k] * B[n, k]
// (minit/operator/linalg.py:29-35, minit/cuda/kernel/cublas.py:83), so both
// operands are K-contiguous -- exactly what the MFMA operand layout wants
// (16 consecutive k per lane).
//
// Tiling: block tile 128 x 256 x 64, eight waves in a 2 x 4 arrangement (two
// per SIMD, so one wave's MFMA issue gaps are filled by the other), each
// computing 64 x 64 as 2 x 2 MFMA tiles of 32 x 32.  Operand tiles travel
// global -> a register ring several k-steps deep -> LDS (double buffered, one
// barrier per 64-k step) -> fragment registers (double buffered per half
// k-step).  LDS rows are 64 bytes; the 16-byte chunk index is XOR-swizzled with
// bits 2..3 of the row, which makes ds_read_b128 of 32 consecutive rows
// conflict-free on the 64-bank LDS.  blockIdx -> tile mapping is XCD-aware:
// consecutive block ids land on different XCDs, so each XCD is given a compact
// rectangle of tiles and its L2 sees each operand row few times.
#include "common.h"

namespace mh {

constexpr int kI8BM = 128, kI8BN = 256, kI8BK = 64, kI8Threads = 512;
constexpr int kI8StagePitch = 144;  // bytes per staged output row: 64 fp16 + 16 bytes of padding

__device__ __forceinline__ int swz(int row, int chunk) { return row * 64 + ((chunk ^ ((row >> 2) & 3)) << 4); }

template <int R>  // k-steps a global load is issued ahead of its use; K / 64 is a multiple of R
__global__ __launch_bounds__(kI8Threads) void i8_gemm_kernel(
    const int8_t* __restrict__ A, const int8_t* __restrict__ W, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, half_t* __restrict__ out, int32_t* __restrict__ acc_out,
    int M, int N, int K, int tiles_m, int tiles_n, int group_m, int xcd_chunk) {
    // [2][A tile | W tile]; reused by the epilogue as eight 32-row output stages
    __shared__ __attribute__((aligned(16))) int8_t smem[2 * (kI8BM + kI8BN) * kI8BK];
    __shared__ float s_a[kI8BM], s_w[kI8BN];
    auto As = [&](int buf) { return smem + buf * (kI8BM + kI8BN) * kI8BK; };
    auto Bs = [&](int buf) { return smem + buf * (kI8BM + kI8BN) * kI8BK + kI8BM * kI8BK; };

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
    const int wy = wave >> 2, wx = wave & 3;
    const int l32 = lane & 31, lh = lane >> 5;

    if (out) {  // visible to the epilogue through the barriers of the main loop
        if (tid < kI8BN) s_w[tid] = w_scale[min(n0 + tid, N - 1)];
        if (tid < kI8BM) s_a[tid] = a_scale[min(m0 + tid, M - 1)];
    }

    // acc[i][j] is the 32 x 32 tile (rows m of A block i, columns n of W block j),
    // computed transposed -- the W fragment is the MFMA's first operand -- so a
    // lane ends up with runs of four consecutive n for one m (see the epilogue).
    int16_t_v acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    // Global -> register ring -> LDS.  A k-step of MFMAs (~0.2 us) is far shorter
    // than a trip to L2/HBM: the operands of k-step kt + R are requested while kt
    // is computed and only stored to LDS R steps later.  Per stage A has 512
    // 16-byte chunks (one per thread) and W has 1024 (two per thread).
    int4_t ra[R], rb[R][2];
    const int crow = tid >> 2, cchunk = tid & 3;
    const int8_t* a_src = A + (size_t)min(m0 + crow, M - 1) * K + cchunk * 16;
    const int8_t* b_src[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) b_src[j] = W + (size_t)min(n0 + crow + 128 * j, N - 1) * K + cchunk * 16;
    const int KT = K / kI8BK;
    auto load_stage = [&](int slot, int kt) {
        const int k0 = min(kt, KT - 1) * kI8BK;
        ra[slot] = *reinterpret_cast<const int4_t*>(a_src + k0);
#pragma unroll
        for (int j = 0; j < 2; ++j) rb[slot][j] = *reinterpret_cast<const int4_t*>(b_src[j] + k0);
    };
    // A stage is written to LDS in two parts, one under each half k-step, so that
    // neither half is heavy on LDS writes (which run at a third of the read rate).
    auto store_part = [&](int part, int slot, int buf) {
        if (part == 0) {
            *reinterpret_cast<int4_t*>(As(buf) + swz(crow, cchunk)) = ra[slot];
        } else {
#pragma unroll
            for (int j = 0; j < 2; ++j)
                *reinterpret_cast<int4_t*>(Bs(buf) + swz(crow + 128 * j, cchunk)) = rb[slot][j];
        }
    };
    // Fragment registers, two sets: the MFMAs of one half k-step (32 k) run
    // while the ds_reads of the next half fill the other set.
    int4_t fa[2][2], fb[2][2];
    auto read_frag = [&](int set, int buf, int ks) {
        const int chunk = ks * 2 + lh;
#pragma unroll
        for (int i = 0; i < 2; ++i)
            fa[set][i] = *reinterpret_cast<const int4_t*>(As(buf) + swz(wy * 64 + i * 32 + l32, chunk));
#pragma unroll
        for (int j = 0; j < 2; ++j)
            fb[set][j] = *reinterpret_cast<const int4_t*>(Bs(buf) + swz(wx * 64 + j * 32 + l32, chunk));
    };
    auto mfma_one = [&](int set, int t) {
        const int i = t >> 1, j = t & 1;
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[set][j], fa[set][i], acc[i][j], 0, 0, 0);
    };

    // Stage s lives in ring slot s % R and LDS buffer s & 1.
#pragma unroll
    for (int r = 0; r < R; ++r) load_stage(r, r);
    store_part(0, 0, 0);
    store_part(1, 0, 0);
    load_stage(0, R);
    __syncthreads();
    read_frag(0, 0, 0);
    store_part(0, 1 % R, 1);
    for (int kt0 = 0; kt0 < KT; kt0 += R) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int kt = kt0 + r;
            const int buf = kt & 1;
            // first half: the rest of stage kt + 1 goes to the other buffer and the
            // second-half fragments are fetched under the first-half MFMAs; the
            // ring slot of stage kt + 1 is then requested again for kt + 1 + R.
            // The first MFMA of each half is issued ahead of the half's LDS traffic
            // so the matrix pipe is never waiting behind a full LDS queue.
            mfma_one(0, 0);
            __builtin_amdgcn_sched_barrier(0);
            store_part(1, (r + 1) % R, buf ^ 1);
            read_frag(1, buf, 1);
            __builtin_amdgcn_sched_barrier(0);
            mfma_one(0, 1);
            mfma_one(0, 2);
            mfma_one(0, 3);
            load_stage((r + 1) % R, kt + 1 + R);
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
            // second half: first-half fragments of stage kt + 1 and the first part
            // of stage kt + 2 (into this stage's buffer, which every wave has
            // finished reading at the barrier) under the second-half MFMAs.
            mfma_one(1, 0);
            __builtin_amdgcn_sched_barrier(0);
            read_frag(0, buf ^ 1, 0);
            store_part(0, (r + 2) % R, buf);
            __builtin_amdgcn_sched_barrier(0);
            mfma_one(1, 1);
            mfma_one(1, 2);
            mfma_one(1, 3);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    __syncthreads();  // every wave is done with the operand buffers

    // Epilogue.  acc[i][j][q * 4 + e] belongs to row m = l32 and column
    // n = q * 8 + lh * 4 + e of its tile: four consecutive n per (lane, q).
    const int wm = wy * 64, wn = wx * 64;  // wave tile origin inside the block tile
    if (acc_out) {
        const bool n_vec = (N % 4 == 0);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int m = m0 + wm + i * 32 + l32;
            if (m >= M) continue;
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int n = n0 + wn + j * 32 + q * 8 + lh * 4;
                    if (n >= N) continue;
                    int32_t* dst = acc_out + (size_t)m * N + n;
                    if (n_vec && n + 4 <= N) {
                        int4_t v = {acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]};
                        *reinterpret_cast<int4_t*>(dst) = v;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (n + e < N) dst[e] = acc[i][j][q * 4 + e];
                    }
                }
        }
    }
    if (out) {
        // Scaled fp16 values are staged per wave as 32 rows x 64 columns in LDS
        // and leave as whole 128-byte row pieces, 16 bytes per lane.
        int8_t* stage = smem + wave * (32 * kI8StagePitch);
        const bool n_vec = (N % 8 == 0);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const float sa = s_a[wm + i * 32 + l32];
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int nl = j * 32 + q * 8 + lh * 4;
                    const float4_t sw = *reinterpret_cast<const float4_t*>(s_w + wn + nl);
                    half4_t h;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        // The scale product and its product with the sum are each
                        // rounded to fp32 and only then to fp16; the empty asm keeps
                        // the compiler from fusing the last two steps into one
                        // mixed-precision instruction that rounds once.
                        float prod = (float)acc[i][j][q * 4 + e] * (sa * sw[e]);
                        asm volatile("" : "+v"(prod));
                        h[e] = (half_t)prod;
                    }
                    *reinterpret_cast<half4_t*>(stage + l32 * kI8StagePitch + nl * 2) = h;
                }
            // wave-private region: only this wave's own LDS traffic has to land
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const int row = rr * 8 + (lane >> 3), c8 = (lane & 7) * 8;
                const int m = m0 + wm + i * 32 + row, n = n0 + wn + c8;
                const int4_t v = *reinterpret_cast<const int4_t*>(stage + row * kI8StagePitch + c8 * 2);
                if (m >= M || n >= N) continue;
                half_t* dst = out + (size_t)m * N + n;
                if (n_vec) {
                    *reinterpret_cast<int4_t*>(dst) = v;
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

// The same tiling with 128-k stages, for K a multiple of 128.  A row of a stage is
// then one whole 128-byte line: with 64-k stages every line is fetched by two
// consecutive k-steps, 24 KiB of half lines per CU and step, and the vector L1
// (smaller than one stage) cannot keep the second halves.  It takes 96 KiB of the
// CU's 160 KiB of LDS, halves the barriers, and splits a k-step into four
// quarters of four MFMAs per wave: the fragments of the next quarter and a sixth
// to a third of the next stage's LDS writes travel under each.
template <int R>  // k-steps a global load is issued ahead of its use; K / 128 is a multiple of R
__global__ __launch_bounds__(kI8Threads) void i8_gemm_k128_kernel(
    const int8_t* __restrict__ A, const int8_t* __restrict__ W, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, half_t* __restrict__ out, int32_t* __restrict__ acc_out,
    int M, int N, int K, int tiles_m, int tiles_n, int group_m, int xcd_chunk) {
    constexpr int BK = 128;
    // [2][A tile | W tile]; reused by the epilogue as eight 32-row output stages
    __shared__ __attribute__((aligned(16))) int8_t smem[2 * (kI8BM + kI8BN) * BK];
    __shared__ float s_a[kI8BM], s_w[kI8BN];
    auto As = [&](int buf) { return smem + buf * (kI8BM + kI8BN) * BK; };
    auto Bs = [&](int buf) { return smem + buf * (kI8BM + kI8BN) * BK + kI8BM * BK; };

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
    const int wy = wave >> 2, wx = wave & 3;
    const int l32 = lane & 31, lh = lane >> 5;

    if (out) {  // visible to the epilogue through the barriers of the main loop
        if (tid < kI8BN) s_w[tid] = w_scale[min(n0 + tid, N - 1)];
        if (tid < kI8BM) s_a[tid] = a_scale[min(m0 + tid, M - 1)];
    }

    // acc[i][j] is the 32 x 32 tile (rows m of A block i, columns n of W block j),
    // computed transposed -- the W fragment is the MFMA's first operand -- so a
    // lane ends up with runs of four consecutive n for one m (see the epilogue).
    int16_t_v acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    // Global -> register ring -> LDS.  Per stage A has 1024 16-byte chunks (two per
    // thread) and W has 2048 (four per thread); eight threads fetch one row's line.
    int4_t ra[R][2], rb[R][4];
    const int crow = tid >> 3, cchunk = tid & 7;
    // buffer loads: a fixed 32-bit offset per thread and row, the k offset scalar
    const __amdgpu_buffer_rsrc_t a_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(A), 0, (int)((size_t)M * K), kBufferRsrcFlags);
    const __amdgpu_buffer_rsrc_t w_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(W), 0, (int)((size_t)N * K), kBufferRsrcFlags);
    int a_off[2], b_off[4];
#pragma unroll
    for (int j = 0; j < 2; ++j) a_off[j] = min(m0 + crow + 64 * j, M - 1) * K + cchunk * 16;
#pragma unroll
    for (int j = 0; j < 4; ++j) b_off[j] = min(n0 + crow + 64 * j, N - 1) * K + cchunk * 16;
    const int KT = K / BK;
    auto load_stage = [&](int slot, int kt) {
        const int k0 = min(kt, KT - 1) * BK;
#pragma unroll
        for (int j = 0; j < 2; ++j)
            ra[slot][j] = __builtin_bit_cast(int4_t, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, a_off[j], k0, 0));
#pragma unroll
        for (int j = 0; j < 4; ++j)
            rb[slot][j] = __builtin_bit_cast(int4_t, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, b_off[j], k0, 0));
    };
    // LDS rows are 128 bytes; the chunk index is XOR-ed with bits 1..3 of the row, so
    // that the 32 rows a fragment read touches spread over all 16-byte bank groups.
    auto swz128 = [](int row, int chunk) { return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4); };
    auto store_a = [&](int slot, int buf) {
#pragma unroll
        for (int j = 0; j < 2; ++j) *reinterpret_cast<int4_t*>(As(buf) + swz128(crow + 64 * j, cchunk)) = ra[slot][j];
    };
    auto store_w = [&](int slot, int buf, int j) {
        *reinterpret_cast<int4_t*>(Bs(buf) + swz128(crow + 64 * j, cchunk)) = rb[slot][j];
    };
    // Fragment registers, two sets: the MFMAs of one quarter k-step (32 k) run
    // while the ds_reads of the next quarter fill the other set.
    int4_t fa[2][2], fb[2][2];
    auto read_frag = [&](int set, int buf, int ks) {
        const int chunk = ks * 2 + lh;
#pragma unroll
        for (int i = 0; i < 2; ++i)
            fa[set][i] = *reinterpret_cast<const int4_t*>(As(buf) + swz128(wy * 64 + i * 32 + l32, chunk));
#pragma unroll
        for (int j = 0; j < 2; ++j)
            fb[set][j] = *reinterpret_cast<const int4_t*>(Bs(buf) + swz128(wx * 64 + j * 32 + l32, chunk));
    };
    auto mfma_one = [&](int set, int t) {
        const int i = t >> 1, j = t & 1;
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[set][j], fa[set][i], acc[i][j], 0, 0, 0);
    };
    auto mfma_rest = [&](int set) {
        mfma_one(set, 1);
        mfma_one(set, 2);
        mfma_one(set, 3);
    };

    // Stage s lives in ring slot s % R and LDS buffer s & 1.  Its A part is written
    // in the last quarter of k-step s - 2 (after that step's barrier, into the
    // buffer stage s - 2 has just been read from), its W part in the first three
    // quarters of k-step s - 1; the barrier before the last quarter of s - 1 makes
    // it visible, and that quarter reads its first fragments.
#pragma unroll
    for (int r = 0; r < R; ++r) load_stage(r, r);
    store_a(0, 0);
#pragma unroll
    for (int j = 0; j < 4; ++j) store_w(0, 0, j);
    load_stage(0, R);
    store_a(1 % R, 1);
    __syncthreads();
    read_frag(0, 0, 0);
    for (int kt0 = 0; kt0 < KT; kt0 += R) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int kt = kt0 + r;
            const int buf = kt & 1;
            const int next = (r + 1) % R;
            // quarter 0
            mfma_one(0, 0);
            __builtin_amdgcn_sched_barrier(0);
            store_w(next, buf ^ 1, 0);
            store_w(next, buf ^ 1, 1);
            read_frag(1, buf, 1);
            __builtin_amdgcn_sched_barrier(0);
            mfma_rest(0);
            __builtin_amdgcn_sched_barrier(0);
            // quarter 1
            mfma_one(1, 0);
            __builtin_amdgcn_sched_barrier(0);
            store_w(next, buf ^ 1, 2);
            read_frag(0, buf, 2);
            __builtin_amdgcn_sched_barrier(0);
            mfma_rest(1);
            __builtin_amdgcn_sched_barrier(0);
            // quarter 2: the ring slot of stage kt + 1 is free after its last store
            mfma_one(0, 0);
            __builtin_amdgcn_sched_barrier(0);
            store_w(next, buf ^ 1, 3);
            read_frag(1, buf, 3);
            __builtin_amdgcn_sched_barrier(0);
            mfma_rest(0);
            load_stage(next, kt + 1 + R);
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
            // quarter 3
            mfma_one(1, 0);
            __builtin_amdgcn_sched_barrier(0);
            read_frag(0, buf ^ 1, 0);
            store_a((r + 2) % R, buf);
            __builtin_amdgcn_sched_barrier(0);
            mfma_rest(1);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    __syncthreads();  // every wave is done with the operand buffers

    // Epilogue.  acc[i][j][q * 4 + e] belongs to row m = l32 and column
    // n = q * 8 + lh * 4 + e of its tile: four consecutive n per (lane, q).
    const int wm = wy * 64, wn = wx * 64;  // wave tile origin inside the block tile
    if (acc_out) {
        const bool n_vec = (N % 4 == 0);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int m = m0 + wm + i * 32 + l32;
            if (m >= M) continue;
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int n = n0 + wn + j * 32 + q * 8 + lh * 4;
                    if (n >= N) continue;
                    int32_t* dst = acc_out + (size_t)m * N + n;
                    if (n_vec && n + 4 <= N) {
                        int4_t v = {acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]};
                        *reinterpret_cast<int4_t*>(dst) = v;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (n + e < N) dst[e] = acc[i][j][q * 4 + e];
                    }
                }
        }
    }
    if (out) {
        // Scaled fp16 values are staged per wave as 32 rows x 64 columns in LDS
        // and leave as whole 128-byte row pieces, 16 bytes per lane.
        int8_t* stage = smem + wave * (32 * kI8StagePitch);
        const bool n_vec = (N % 8 == 0);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const float sa = s_a[wm + i * 32 + l32];
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int nl = j * 32 + q * 8 + lh * 4;
                    const float4_t sw = *reinterpret_cast<const float4_t*>(s_w + wn + nl);
                    half4_t h;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        // The scale product and its product with the sum are each
                        // rounded to fp32 and only then to fp16; the empty asm keeps
                        // the compiler from fusing the last two steps into one
                        // mixed-precision instruction that rounds once.
                        float prod = (float)acc[i][j][q * 4 + e] * (sa * sw[e]);
                        asm volatile("" : "+v"(prod));
                        h[e] = (half_t)prod;
                    }
                    *reinterpret_cast<half4_t*>(stage + l32 * kI8StagePitch + nl * 2) = h;
                }
            // wave-private region: only this wave's own LDS traffic has to land
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const int row = rr * 8 + (lane >> 3), c8 = (lane & 7) * 8;
                const int m = m0 + wm + i * 32 + row, n = n0 + wn + c8;
                const int4_t v = *reinterpret_cast<const int4_t*>(stage + row * kI8StagePitch + c8 * 2);
                if (m >= M || n >= N) continue;
                half_t* dst = out + (size_t)m * N + n;
                if (n_vec) {
                    *reinterpret_cast<int4_t*>(dst) = v;
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

// i8_gemm_dma.hip: the same tiling with operand tiles loaded straight into LDS
bool i8_gemm_dma_supported(int M, int N, int K);
int i8_gemm_dma_launch(hipStream_t stream, const int8_t* a, const int8_t* w, const float* a_scale,
                       const float* w_scale, void* out_f16, int32_t* acc_i32, int M, int N, int K);

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
    MH_REQUIRE(((uintptr_t)a | (uintptr_t)w | (uintptr_t)acc_i32) % 16 == 0 && (uintptr_t)out_f16 % 16 == 0,
               "mh_i8_gemm: operands and outputs must be 16-byte aligned");
    const int tiles_m = (M + kI8BM - 1) / kI8BM, tiles_n = (N + kI8BN - 1) / kI8BN;
    const int tiles = tiles_m * tiles_n;
    const int group_m = tiles_m < 8 ? tiles_m : 8;
    const int xcd_chunk = (tiles % 8 == 0) ? tiles / 8 : 0;
    if (i8_gemm_dma_supported(M, N, K))
        return i8_gemm_dma_launch(as_stream(stream), a, w, a_scale, w_scale, out_f16, acc_i32, M, N, K);
    static const char* no128 = getenv("MH_I8_NO_K128");
    // the 128-k kernel addresses its operands with 32-bit buffer offsets
    if (K % 128 == 0 && (size_t)M * K < ((size_t)1 << 31) && (size_t)N * K < ((size_t)1 << 31) &&
        !(no128 && *no128 && atoi(no128))) {
        const int kt128 = K / 128;
#define MH_I8_LAUNCH128(R)                                                                                          \
    hipLaunchKernelGGL(i8_gemm_k128_kernel<R>, dim3(tiles), dim3(kI8Threads), 0, as_stream(stream), a, w, a_scale, \
                       w_scale, (half_t*)out_f16, acc_i32, M, N, K, tiles_m, tiles_n, group_m, xcd_chunk)
        if (kt128 % 4 == 0) {
            MH_I8_LAUNCH128(4);
        } else if (kt128 % 2 == 0) {
            MH_I8_LAUNCH128(2);
        } else {
            MH_I8_LAUNCH128(1);
        }
#undef MH_I8_LAUNCH128
        MH_CHECK_LAUNCH();
        return MH_OK;
    }
    const int kt = K / kI8BK;
#define MH_I8_LAUNCH(R)                                                                                      \
    hipLaunchKernelGGL(i8_gemm_kernel<R>, dim3(tiles), dim3(kI8Threads), 0, as_stream(stream), a, w, a_scale, w_scale, \
                       (half_t*)out_f16, acc_i32, M, N, K, tiles_m, tiles_n, group_m, xcd_chunk)
    if (kt % 4 == 0) {
        MH_I8_LAUNCH(4);
    } else if (kt % 2 == 0) {
        MH_I8_LAUNCH(2);
    } else {
        MH_I8_LAUNCH(1);
    }
#undef MH_I8_LAUNCH
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
