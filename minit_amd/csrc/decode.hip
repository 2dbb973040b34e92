// Llama-family GPTQ decode step: the callers on either side of the quantized
// linears (examples/llama3_70b.py:77-162,215-249 of the reference), run as one
// native loop that enqueues every kernel of a token step from C++.
//
// What differs from the reference's step, by design:
//   * KV cache is preallocated [B, KVH, T, D] and appended in place; the
//     reference re-allocates and concatenates it every token (llama3_70b.py:97-100)
//     and stores it expanded to all query heads (:164-168).
//   * attention for one new token is a split-KV streaming kernel that fuses the
//     1/sqrt(d) scale, softmax and the P.V product; grouped-query heads that
//     share a KV head are processed together so K and V are read once.
//   * residual add + RMSNorm, RoPE + cache append, SiLU*up are fused kernels.
//   * sampling is an on-device argmax (the reference copies the logits to the
//     host, minit/chat/sample.py:11-14).
#include "gptq_common.h"

#include <cstring>
#include <new>
#include <vector>

namespace mh {

int gptq_matmul_dispatch(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                         const void* scales, void* out, int M, int N, int K, int group_size, int bits,
                         void* workspace, size_t workspace_bytes);
bool gemm_silu_pairs_supported(int M, int N, int K, int group_size, int bits);
bool gemm_norm_fusion_supported(int M, int N, int K, int group_size, int bits, int epilogue);
int gemm_residual_ssq_pieces(int M, int N, int K, int group_size, int bits);
int gptq_matmul_fused(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                      const void* scales, void* out, int M, int N, int K, int group_size, int bits,
                      void* workspace, size_t workspace_bytes, int epilogue, const SmallFuse& fuse);
int gptq_matmul_silu_pairs(hipStream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                           const void* scales, void* out, int M, int N, int K, int group_size, int bits,
                           void* workspace, size_t workspace_bytes);

// ---- small fused kernels --------------------------------------------------------------------------

__global__ __launch_bounds__(256) void embed_gather_kernel(const int32_t* __restrict__ tokens,
                                                           const half_t* __restrict__ embed,
                                                           half_t* __restrict__ out, int hidden, int vocab) {
    const int b = blockIdx.x;
    int tok = tokens[b];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    const uint4* src = reinterpret_cast<const uint4*>(embed + (size_t)tok * hidden);
    uint4* dst = reinterpret_cast<uint4*>(out + (size_t)b * hidden);
    for (int i = threadIdx.x; i < hidden / 8; i += blockDim.x) dst[i] = src[i];
}

// h <- fp16(h + delta) (skipped when delta == nullptr); xn <- rmsnorm(h) * w.
// The sum is rounded to fp16 before it is normalised, as the separate add and
// norm kernels of the reference would (llama3_70b.py:159-162).
__global__ __launch_bounds__(256) void add_rms_norm_kernel(half_t* __restrict__ h, const half_t* __restrict__ delta,
                                                           const half_t* __restrict__ w, half_t* __restrict__ xn,
                                                           int hidden, float eps) {
    __shared__ float smem[16];
    const size_t row = blockIdx.x;
    uint4* hp = reinterpret_cast<uint4*>(h + row * hidden);
    const uint4* dp = delta ? reinterpret_cast<const uint4*>(delta + row * hidden) : nullptr;
    const uint4* wp = reinterpret_cast<const uint4*>(w);
    uint4* op = reinterpret_cast<uint4*>(xn + row * hidden);
    const int nvec = hidden / 8;
    half8_t vals[4];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int v = c * 256 + threadIdx.x;
        if (v < nvec) {
            half8_t a = __builtin_bit_cast(half8_t, hp[v]);
            if (dp) {
                a = a + __builtin_bit_cast(half8_t, dp[v]);  // fp16 add, one rounding
                hp[v] = __builtin_bit_cast(uint4, a);
            }
            vals[c] = a;
#pragma unroll
            for (int i = 0; i < 8; ++i) ss += (float)a[i] * (float)a[i];
        }
    }
    ss = block_sum(ss, smem);
    const float rms = sqrtf(ss / (float)hidden + eps);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int v = c * 256 + threadIdx.x;
        if (v < nvec) {
            const half8_t wv = __builtin_bit_cast(half8_t, wp[v]);
            half8_t o;
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] = (half_t)((float)vals[c][i] / rms * (float)wv[i]);
            op[v] = __builtin_bit_cast(uint4, o);
        }
    }
}

// h <- fp16(h + delta) only (after the last block).
__global__ void add_kernel(half_t* __restrict__ h, const half_t* __restrict__ delta, size_t n8) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    uint4* hp = reinterpret_cast<uint4*>(h);
    const uint4* dp = reinterpret_cast<const uint4*>(delta);
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += stride) {
        const half8_t a = __builtin_bit_cast(half8_t, hp[i]) + __builtin_bit_cast(half8_t, dp[i]);
        hp[i] = __builtin_bit_cast(uint4, a);
    }
}

// qkv [B, (QH + 2 KVH) * D]: rotate q heads into q_out [B, QH, D]; rotate k
// heads and copy v heads into the caches at positions[b] (V tiled, vt_offset).  One 64-thread block
// per (head, batch row); thread i owns the interleaved pair i
// (minit/cuda/kernel/cuda/rope.py:58-73).
__global__ __launch_bounds__(64) void rope_kv_append_kernel(
    const half_t* __restrict__ qkv, const float* __restrict__ freqs_cos, const float* __restrict__ freqs_sin,
    const int32_t* __restrict__ positions, half_t* __restrict__ q_out, half_t* __restrict__ k_cache,
    half_t* __restrict__ v_cache, int qh, int kvh, int head_dim, int max_seq) {
    const int head = blockIdx.x, b = blockIdx.y;
    const int half_dim = head_dim / 2;
    const int pos = min(max(positions[b], 0), max_seq - 1);  // a full cache overwrites its last slot rather than its neighbour
    const half_t* src = qkv + ((size_t)b * (qh + 2 * kvh) + head) * head_dim;
    for (int i = threadIdx.x; i < half_dim; i += blockDim.x) {
        const float re = (float)src[2 * i], im = (float)src[2 * i + 1];
        if (head >= qh + kvh) {  // v: plain copy
            // the V cache is tiled, [B, KVH, T / 64, D, 64]: see vt_offset
            half_t* dst = v_cache + ((size_t)b * kvh + (head - qh - kvh)) * head_dim * max_seq + vt_offset(2 * i, pos, head_dim);
            dst[0] = src[2 * i];
            dst[kVTile] = src[2 * i + 1];
            continue;
        }
        const float c = freqs_cos[(size_t)pos * half_dim + i], s = freqs_sin[(size_t)pos * half_dim + i];
        const half_t o0 = (half_t)(re * c - im * s), o1 = (half_t)(im * c + re * s);
        half_t* dst = head < qh ? q_out + ((size_t)b * qh + head) * head_dim
                                : k_cache + (((size_t)b * kvh + (head - qh)) * max_seq + pos) * head_dim;
        dst[2 * i] = o0;
        dst[2 * i + 1] = o1;
    }
}

// act[b, t*128 + c] = silu(gu[b, t*256 + c]) * gu[b, t*256 + 128 + c] (gate and up
// interleaved in blocks of 128 columns); fp32 until the store.  Only used when the
// product kernel cannot apply this epilogue itself.
__global__ void silu_mul_fused_kernel(const half_t* __restrict__ gu, half_t* __restrict__ act, int batch, int ffn) {
    const size_t n8 = (size_t)batch * ffn / 8;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const int row8 = ffn / 8;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += stride) {
        const size_t b = i / row8, c = i % row8;   // c: 8-column chunk of the output row
        const half_t* gp = gu + b * 2 * ffn + c / 16 * 256 + c % 16 * 8;
        const half8_t g = __builtin_bit_cast(half8_t, *reinterpret_cast<const uint4*>(gp));
        const half8_t u = __builtin_bit_cast(half8_t, *reinterpret_cast<const uint4*>(gp + 128));
        half8_t o;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float gf = (float)g[e];
            o[e] = (half_t)(gf / (1.f + expf(-gf)) * (float)u[e]);
        }
        reinterpret_cast<uint4*>(act)[i] = __builtin_bit_cast(uint4, o);
    }
}

int silu_pairs_launch(hipStream_t stream, const void* gate_up, void* out, int rows, int ffn) {
    const size_t n8 = (size_t)rows * ffn / 8;
    size_t grid = (n8 + 255) / 256;
    const size_t cap = (size_t)compute_units() * 16;
    if (grid > cap) grid = cap;
    hipLaunchKernelGGL(silu_mul_fused_kernel, dim3((unsigned)grid), dim3(256), 0, stream, (const half_t*)gate_up,
                       (half_t*)out, rows, ffn);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

// token[b] = argmax_v logits[b, v] (first maximum); appended to the output
// stream and fed back as the next input; positions[b] += 1.  out_tokens points
// at this step's row of the output, or, when pos_base is given, at the whole
// [steps, batch] output and the row is positions[b] - pos_base[b]: the same
// launch, replayed, then fills one row after the other.
__global__ __launch_bounds__(1024) void argmax_advance_kernel(const half_t* __restrict__ logits,
                                                              int32_t* __restrict__ tokens,
                                                              int32_t* __restrict__ out_tokens,
                                                              int32_t* __restrict__ positions,
                                                              const int32_t* __restrict__ pos_base, int vocab) {
    __shared__ float sval[16];
    __shared__ int sidx[16];
    const int b = blockIdx.x;
    const half_t* row = logits + (size_t)b * vocab;
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    auto consider = [&](float x, int v) {
        if (x > best || (x == best && v < best_i)) {
            best = x;
            best_i = v;
        }
    };
    const bool aligned = ((uintptr_t)row % 16) == 0;
    const int nvec = aligned ? vocab / 8 : 0;
    for (int i = threadIdx.x; i < nvec; i += blockDim.x) {
        const half8_t v = __builtin_bit_cast(half8_t, reinterpret_cast<const uint4*>(row)[i]);
#pragma unroll
        for (int e = 0; e < 8; ++e) consider((float)v[e], i * 8 + e);
    }
    for (int v = nvec * 8 + threadIdx.x; v < vocab; v += blockDim.x) consider((float)row[v], v);
    // wave reduction, then across the 16 waves
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float o = __shfl_xor(best, off, 64);
        const int oi = __shfl_xor(best_i, off, 64);
        consider(o, oi);
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) {
        sval[wave] = best;
        sidx[wave] = best_i;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); ++w) consider(sval[w], sidx[w]);
        const int tok = best_i == 0x7fffffff ? 0 : best_i;
        tokens[b] = tok;
        const int pos = positions ? positions[b] : 0;  // no positions: a plain row-wise argmax
        if (out_tokens) out_tokens[pos_base ? (size_t)(pos - pos_base[b]) * gridDim.x + b : (size_t)b] = tok;
        if (positions) positions[b] = pos + 1;
    }
}

// ---- split-KV decode attention ---------------------------------------------------------------------
// One block per (split, kv head, batch row); the G query heads that share the KV
// head are the (padded to 16) rows of fp16 MFMA tiles.  Per 64-position chunk a
// wave computes S = Q K^T with 16 v_mfma_f32_16x16x32_f16 (K rows are
// d-contiguous, which is the B-operand layout as loaded), does the running
// max / sum softmax on the accumulator layout, passes P through LDS to turn it
// into an A operand, and accumulates O += P V with 16 more MFMAs.  For that
// product the B operand needs eight consecutive positions of one dim per lane,
// so V is cached with positions contiguous, in tiles of 64, [B, KVH, T / 64, D, 64]
// (vt_offset: a chunk of a wave is one tile).  Waves own
// alternate chunks and are merged through LDS; splits are merged by the last
// block to arrive.

template <int G, int D, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void attn_decode_kernel(
    const half_t* __restrict__ q, const half_t* __restrict__ k_cache, const half_t* __restrict__ vt_cache,
    const int32_t* __restrict__ positions, half_t* __restrict__ out, float* partial, unsigned* counters,
    int kvh, int max_seq, float scale, int splits) {
    static_assert(D == 128 && G <= 16, "head size 128, at most 16 query heads per KV head");
    constexpr int PP = 72;  // halfs per row of the P tile in LDS (64 + padding)
    const int split = blockIdx.x, g = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int i16 = lane & 15, kq = lane >> 4;
    // Chunks of 64 positions (one tile of the V cache) are dealt round robin, first over the
    // blocks of a (row, KV head) pair and then over their waves: chunk c belongs to block
    // c % splits, wave (c / splits) % WAVES.  The deal does not depend on the length, so a
    // wave requests its first chunk before the position has arrived, and no wave holds more
    // than one chunk over the others.
    const int stride = splits * WAVES * 64;
    const int c_first = (split + wave * splits) * 64;
    const int t1 = min(max(positions[b], 0), max_seq - 1) + 1;  // the new token has been appended

    __shared__ __attribute__((aligned(16))) half_t p_s[WAVES][16 * PP];
    __shared__ float m_s[WAVES][16], l_s[WAVES][16];
    __shared__ float acc_s[WAVES][G][D];

    // A operand of S = Q K^T: row = head i16, k = dims s*32 + kq*8 .. +8
    uint4 qf[4];
    {
        const half_t* qp = q + (((size_t)b * kvh + g) * G + min(i16, G - 1)) * D + kq * 8;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            qf[s] = *reinterpret_cast<const uint4*>(qp + s * 32);
            if (i16 >= G) qf[s] = make_uint4(0, 0, 0, 0);
        }
    }
    const half_t* kbase = k_cache + ((size_t)b * kvh + g) * max_seq * D;
    const half_t* vbase = vt_cache + ((size_t)b * kvh + g) * D * max_seq;

    // rows of every accumulator tile held by this lane: heads kq*4 + r
    float m_run[4], l_run[4];
    float4_t acc[8];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        m_run[r] = -INFINITY;
        l_run[r] = 0.f;
    }
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) acc[dt] = float4_t{0.f, 0.f, 0.f, 0.f};

    // all loads of a chunk are issued before the first use (refilling K after Q K^T and V
    // after P V for the wave's next chunk, so that loads stay in flight under the arithmetic,
    // measured no faster at batch 1 and 32 and slower at 8).  Rows and tiles are clamped to
    // the cache, not to the length: what lies past the end is masked below.
    uint4 kf[4][4], vf[8][2];
    auto load_chunk = [&](int c0) {
#pragma unroll
        for (int pt = 0; pt < 4; ++pt) {
            const int row = min(c0 + pt * 16 + i16, max_seq - 1);
            const half_t* kp = kbase + (size_t)row * D + kq * 8;
#pragma unroll
            for (int s = 0; s < 4; ++s) kf[pt][s] = *reinterpret_cast<const uint4*>(kp + s * 32);
        }
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int p0 = min(c0 + ks * 32 + kq * 8, max_seq - 8);
#pragma unroll
            for (int dt = 0; dt < 8; ++dt)
                vf[dt][ks] = *reinterpret_cast<const uint4*>(vbase + vt_offset(dt * 16 + i16, p0));
        }
    };
    load_chunk(c_first);
    // Two waves share a SIMD when a block has eight, and the older one wins every arbitration: the
    // priority of a wave falls with the share of its chunks it has behind it, so that the four
    // younger waves are not left to walk their last chunks alone.
    const int n_chunks = t1 > c_first ? (t1 - c_first + stride - 1) / stride : 0;
    int chunk_no = 0;
    for (int c0 = c_first; c0 < t1;) {
        if constexpr (WAVES > 4) {
            set_priority_by_progress(chunk_no++, n_chunks);
        }
        // S tile pt: rows = heads kq*4 + r, column = position c0 + pt*16 + i16
        float4_t sc[4];
#pragma unroll
        for (int pt = 0; pt < 4; ++pt) {
            sc[pt] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 4; ++s)
                sc[pt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, qf[s]),
                                                                __builtin_bit_cast(half8_t, kf[pt][s]), sc[pt], 0, 0, 0);
        }
        float alpha[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float mx = -INFINITY;
#pragma unroll
            for (int pt = 0; pt < 4; ++pt) {
                const bool valid = c0 + pt * 16 + i16 < t1;
                sc[pt][r] = valid ? sc[pt][r] * scale : -INFINITY;
                mx = fmaxf(mx, sc[pt][r]);
            }
#pragma unroll
            for (int off = 1; off < 16; off <<= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
            const float m_new = fmaxf(m_run[r], mx);  // finite: every chunk holds a valid position
            alpha[r] = expf(m_run[r] - m_new);         // exp(-inf) = 0 on the first chunk
            float sum = 0.f;
#pragma unroll
            for (int pt = 0; pt < 4; ++pt) {
                const float pv = expf(sc[pt][r] - m_new);  // exp(-inf) = 0 for masked positions
                sum += pv;
                p_s[wave][(kq * 4 + r) * PP + pt * 16 + i16] = (half_t)pv;
            }
#pragma unroll
            for (int off = 1; off < 16; off <<= 1) sum += __shfl_xor(sum, off, 64);
            l_run[r] = l_run[r] * alpha[r] + sum;
            m_run[r] = m_new;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // A operand of O += P V: row = head i16, k = positions ks*32 + kq*8 .. +8 of the chunk
        uint4 pa[2];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
            pa[ks] = *reinterpret_cast<const uint4*>(&p_s[wave][i16 * PP + ks * 32 + kq * 8]);
        if (c0 + 64 > t1) {
            // positions past the end carry weight 0 but whatever the cache holds there
            // (possibly not finite): clear them
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const int p0 = c0 + ks * 32 + kq * 8;
#pragma unroll
                for (int dt = 0; dt < 8; ++dt) {
                    half8_t v = __builtin_bit_cast(half8_t, vf[dt][ks]);
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (p0 + e >= t1) v[e] = (half_t)0.f;
                    vf[dt][ks] = __builtin_bit_cast(uint4, v);
                }
            }
        }
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) {
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[dt][r] *= alpha[r];
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
                acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, pa[ks]),
                                                                 __builtin_bit_cast(half8_t, vf[dt][ks]), acc[dt], 0, 0, 0);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();  // p_s is rewritten by the next chunk
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        c0 += stride;
        if (c0 < t1) load_chunk(c0);
    }

    // acc[dt][r] is head kq*4 + r, dim dt*16 + i16
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int h = kq * 4 + r;
        if (h < G) {
#pragma unroll
            for (int dt = 0; dt < 8; ++dt) acc_s[wave][h][dt * 16 + i16] = acc[dt][r];
            if (i16 == 0) {
                m_s[wave][h] = m_run[r];
                l_s[wave][h] = l_run[r];
            }
        }
    }
    __syncthreads();

    // merge the waves: thread -> (head, four dims)
    constexpr int REC = D + 4;        // floats per (head, split) record: acc[D], m, l, two unused
    constexpr int ITEMS = G * D / 4;  // <= 256
    const size_t head0 = ((size_t)b * kvh + g) * G;
    const int h = tid / (D / 4), d = tid % (D / 4) * 4;
    if (tid < ITEMS) {
        float mm = m_s[0][h];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) mm = fmaxf(mm, m_s[w][h]);
        float ll = 0.f;
        float4_t a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float f = (m_s[w][h] == -INFINITY) ? 0.f : expf(m_s[w][h] - mm);
            ll += l_s[w][h] * f;
            a += *reinterpret_cast<const float4_t*>(&acc_s[w][h][d]) * f;
        }
        if (splits == 1) {
            const half4_t o = {(half_t)(a[0] / ll), (half_t)(a[1] / ll), (half_t)(a[2] / ll), (half_t)(a[3] / ll)};
            *reinterpret_cast<half4_t*>(out + (head0 + h) * D + d) = o;
        } else {
            float* pp = partial + ((head0 + h) * splits + split) * REC;
            store_agent4(pp + d, a);
            if (d == 0) store_agent4(pp + D, float4_t{mm, ll, 0.f, 0.f});
        }
    }
    if (splits == 1) return;

    __shared__ int is_last;
    if (!arrive_and_check_last(counters + (size_t)b * kvh + g, (unsigned)splits, &is_last)) return;
    // Last block: merge the splits.  Every thread folds the splits of its four
    // output elements with the running-maximum recurrence, reading each split's
    // maximum, sum and partial values itself: the loads of up to 16 splits are
    // independent and in flight together, so the merge costs one memory round
    // trip.
    constexpr int BATCH = 16;
    if (tid < ITEMS) {
        const float* pp = partial + (head0 + h) * splits * REC;
        float mm = -INFINITY, ll = 0.f;
        float4_t a = {0.f, 0.f, 0.f, 0.f};
        for (int sp0 = 0; sp0 < splits; sp0 += BATCH) {
            float ms[BATCH], ls[BATCH];
            float4_t as[BATCH];
#pragma unroll
            for (int u = 0; u < BATCH; ++u) {
                const float* ps = pp + (size_t)min(sp0 + u, splits - 1) * REC;
                as[u] = load_agent4(ps + d);
                ms[u] = load_agent(ps + D);
                ls[u] = load_agent(ps + D + 1);
            }
            wait_agent_loads(as);
#pragma unroll
            for (int u = 0; u < BATCH; ++u) {
                if (sp0 + u < splits && ms[u] != -INFINITY) {
                    const float m_new = fmaxf(mm, ms[u]);
                    const float f_old = expf(mm - m_new);  // exp(-inf) = 0 for the first split folded in
                    const float f = expf(ms[u] - m_new);
                    ll = ll * f_old + ls[u] * f;
                    a = a * f_old + as[u] * f;
                    mm = m_new;
                }
            }
        }
        const half4_t o = {(half_t)(a[0] / ll), (half_t)(a[1] / ll), (half_t)(a[2] / ll), (half_t)(a[3] / ll)};
        *reinterpret_cast<half4_t*>(out + (head0 + h) * D + d) = o;
    }
}

// ---- model description and the decode loop ------------------------------------------------------------

struct Llama {
    mh_llama_config cfg;
    std::vector<mh_llama_layer> layers;
    const void* embed = nullptr;
    const void* lm_head = nullptr;
    const void* final_norm = nullptr;
    const float* cos = nullptr;
    const float* sin = nullptr;
    // one recorded decode step per set of buffers it was recorded on
    struct StepGraph {
        int batch;
        const void *tokens, *positions, *out_tokens, *scratch;
        hipGraphExec_t exec;
    };
    std::vector<StepGraph> graphs;
    void drop_graphs() {
        for (auto& g : graphs) (void)hipGraphExecDestroy(g.exec);
        graphs.clear();
    }
};

struct Scratch {
    half_t *h, *xn, *qkv, *q, *attn, *delta, *gu, *act, *logits;
    half_t* gathered;  // activations in the row order of an act-order weight (mh_qlinear::perm)
    float* attn_partial;
    float *ssq_a, *ssq_b;  // per-piece sums of squares of the residual stream, [batch, at most hidden / 32]
    int32_t* pos_base;     // positions at the start of a call that replays a recorded step
    unsigned* attn_counters;
    unsigned* norm_clamped;  // one word, set when a fused norm's h * w left the fp16 range (never cleared by the loop)
    void* gptq_ws;
    size_t gptq_ws_bytes;
    size_t total;
};

static size_t align_up(size_t v) { return (v + 255) / 256 * 256; }

// Blocks of a (row, KV head) pair.  A CU sustains about 90 KB of cache reads in flight whatever
// the number of waves asking, so a second block on a CU doubles that CU's time: the launch
// takes as many blocks as there are CUs and no more (measured at context 2048, batch 2 to 24:
// 192 to 256 blocks are the fastest launch at every batch size, 288 and more are 15 to 40 %
// slower), and not more than one 64-position chunk per wave needs.  A pair that is left with
// one block runs eight waves instead of four and merges nothing across blocks.
static int attn_splits(int n_kv_heads, int max_seq, int batch) {
    const int pairs = batch * n_kv_heads;
    const int chunks = (max_seq + 63) / 64;
    int splits = (chunks + 3) / 4;
    const int cap = compute_units() / pairs;
    if (splits > cap) splits = cap;
    if (splits > 64) splits = 64;
    static const char* env = getenv("MH_ATTN_SPLITS");
    if (env && *env && atoi(env) > 0) splits = atoi(env) > 64 ? 64 : atoi(env);
    return splits < 1 ? 1 : splits;
}
static int attn_splits(const Llama& m, int batch) { return attn_splits(m.cfg.n_kv_heads, m.cfg.max_seq, batch); }

// Workspace of a stand-alone attention call: arrival counters (one per row and KV
// head, zero between calls), then the per-split records.
static size_t attn_counter_bytes(int batch, int n_kv_heads) { return align_up((size_t)batch * n_kv_heads * sizeof(unsigned)); }
static size_t attn_workspace_bytes(int batch, int n_q_heads, int n_kv_heads, int head_dim, int max_seq) {
    return attn_counter_bytes(batch, n_kv_heads) +
           align_up((size_t)batch * n_q_heads * attn_splits(n_kv_heads, max_seq, batch) * (head_dim + 4) * sizeof(float));
}

template <int G>
static void launch_attn_raw(hipStream_t st, const half_t* q, const half_t* k_cache, const half_t* vt_cache,
                            const int32_t* positions, half_t* out, float* partial, unsigned* counters, int batch,
                            int n_kv_heads, int max_seq, int splits) {
    if (splits == 1)
        hipLaunchKernelGGL((attn_decode_kernel<G, 128, 8>), dim3(1, n_kv_heads, batch), dim3(512), 0, st, q, k_cache,
                           vt_cache, positions, out, partial, counters, n_kv_heads, max_seq, 1.0f / sqrtf(128.f), 1);
    else
        hipLaunchKernelGGL((attn_decode_kernel<G, 128, 4>), dim3(splits, n_kv_heads, batch), dim3(256), 0, st, q,
                           k_cache, vt_cache, positions, out, partial, counters, n_kv_heads, max_seq,
                           1.0f / sqrtf(128.f), splits);
}

static Scratch carve(const Llama& m, int batch, char* base) {
    const mh_llama_config& c = m.cfg;
    const size_t qkv_n = (size_t)(c.n_q_heads + 2 * c.n_kv_heads) * c.head_dim;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        char* p = base ? base + off : nullptr;
        off += align_up(bytes);
        return p;
    };
    Scratch s;
    // counters first: they must start (and are left) zero
    s.attn_counters = (unsigned*)take((size_t)batch * c.n_kv_heads * sizeof(unsigned));
    s.norm_clamped = (unsigned*)take(sizeof(unsigned));
    size_t ws = 0;
    const int shapes[4][2] = {{c.hidden, (int)qkv_n}, {c.n_q_heads * c.head_dim, c.hidden},
                              {c.hidden, 2 * c.ffn}, {c.ffn, c.hidden}};
    for (auto& sh : shapes) {
        const size_t need = mh_gptq_workspace_bytes(batch, sh[1], sh[0], c.group_size, c.bits);
        if (need > ws) ws = need;
    }
    s.gptq_ws_bytes = align_up(ws > 0 ? ws : 256);
    s.gptq_ws = take(s.gptq_ws_bytes);
    s.h = (half_t*)take((size_t)batch * c.hidden * 2);
    s.xn = (half_t*)take((size_t)batch * c.hidden * 2);
    s.qkv = (half_t*)take((size_t)batch * qkv_n * 2);
    s.q = (half_t*)take((size_t)batch * c.n_q_heads * c.head_dim * 2);
    s.attn = (half_t*)take((size_t)batch * c.n_q_heads * c.head_dim * 2);
    s.delta = (half_t*)take((size_t)batch * c.hidden * 2);
    s.gu = (half_t*)take((size_t)batch * 2 * c.ffn * 2);
    s.act = (half_t*)take((size_t)batch * c.ffn * 2);
    s.logits = (half_t*)take((size_t)batch * c.vocab * 2);
    {
        size_t widest = (size_t)c.hidden;
        if ((size_t)c.n_q_heads * c.head_dim > widest) widest = (size_t)c.n_q_heads * c.head_dim;
        if ((size_t)c.ffn > widest) widest = (size_t)c.ffn;
        s.gathered = (half_t*)take((size_t)batch * widest * 2);
    }
    s.attn_partial = (float*)take((size_t)batch * c.n_q_heads * attn_splits(m, batch) * (c.head_dim + 4) * 4);
    s.ssq_a = (float*)take((size_t)batch * ((c.hidden + 31) / 32) * 4);
    s.ssq_b = (float*)take((size_t)batch * ((c.hidden + 31) / 32) * 4);
    s.pos_base = (int32_t*)take((size_t)batch * sizeof(int32_t));
    s.total = off;
    return s;
}

template <int G>
static void launch_attn(hipStream_t st, const Llama& m, const Scratch& s, const mh_llama_layer& L,
                        const int32_t* positions, int batch, int splits) {
    const mh_llama_config& c = m.cfg;
    launch_attn_raw<G>(st, s.q, (const half_t*)L.k_cache, (const half_t*)L.v_cache, positions, s.attn, s.attn_partial,
                       s.attn_counters, batch, c.n_kv_heads, c.max_seq, splits);
}

}  // namespace mh

using namespace mh;

extern "C" {

size_t mh_attn_decode_workspace_bytes(int batch, int n_q_heads, int n_kv_heads, int head_dim, int max_seq) {
    if (batch <= 0 || n_q_heads <= 0 || n_kv_heads <= 0 || head_dim != 128 || max_seq <= 0) return 0;
    return attn_workspace_bytes(batch, n_q_heads, n_kv_heads, head_dim, max_seq);
}

int mh_attn_decode(mh_stream_t stream, const void* q, const void* k_cache, const void* vt_cache,
                   const int32_t* positions, void* out, int batch, int n_q_heads, int n_kv_heads, int head_dim,
                   int max_seq, void* workspace, size_t workspace_bytes) {
    MH_REQUIRE(batch >= 0, "mh_attn_decode: bad batch %d", batch);
    if (batch == 0) return MH_OK;
    MH_REQUIRE(q && k_cache && vt_cache && positions && out, "mh_attn_decode: null pointer");
    MH_REQUIRE(head_dim == 128, "mh_attn_decode: head_dim must be 128, got %d", head_dim);
    MH_REQUIRE(n_kv_heads > 0 && n_q_heads % n_kv_heads == 0, "mh_attn_decode: bad head counts %d / %d", n_q_heads,
               n_kv_heads);
    const int g = n_q_heads / n_kv_heads;
    MH_REQUIRE(g == 1 || g == 2 || g == 4 || g == 8, "mh_attn_decode: %d query heads per KV head unsupported", g);
    MH_REQUIRE(max_seq >= kVTile && max_seq % kVTile == 0, "mh_attn_decode: max_seq must be a multiple of 64, got %d", max_seq);
    MH_REQUIRE(((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)vt_cache | (uintptr_t)out) % 16 == 0,
               "mh_attn_decode: operands must be 16-byte aligned");
    const size_t need = attn_workspace_bytes(batch, n_q_heads, n_kv_heads, head_dim, max_seq);
    if (workspace == nullptr || workspace_bytes < need)
        return fail(MH_ERR_WORKSPACE, "mh_attn_decode: workspace of %zu bytes required, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    MH_REQUIRE((uintptr_t)workspace % 256 == 0, "mh_attn_decode: workspace must be 256-byte aligned");
    unsigned* counters = reinterpret_cast<unsigned*>(workspace);
    float* partial = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + attn_counter_bytes(batch, n_kv_heads));
    const int splits = attn_splits(n_kv_heads, max_seq, batch);
    hipStream_t st = as_stream(stream);
#define MH_ATTN(G)                                                                                                 \
    launch_attn_raw<G>(st, (const half_t*)q, (const half_t*)k_cache, (const half_t*)vt_cache, positions, (half_t*)out, \
                       partial, counters, batch, n_kv_heads, max_seq, splits)
    switch (g) {
        case 1: MH_ATTN(1); break;
        case 2: MH_ATTN(2); break;
        case 4: MH_ATTN(4); break;
        default: MH_ATTN(8); break;
    }
#undef MH_ATTN
    MH_CHECK_LAUNCH();
    return MH_OK;
}

int mh_add_rms_norm(mh_stream_t stream, void* h, const void* delta, const void* weight, void* out, int rows,
                    int hidden, float eps) {
    MH_REQUIRE(rows >= 0 && hidden > 0, "mh_add_rms_norm: bad shape %d x %d", rows, hidden);
    if (rows == 0) return MH_OK;
    MH_REQUIRE(h && weight && out, "mh_add_rms_norm: null pointer");
    MH_REQUIRE(hidden % 8 == 0 && hidden <= 8192, "mh_add_rms_norm: hidden must be a multiple of 8 up to 8192, got %d",
               hidden);
    MH_REQUIRE(((uintptr_t)h | (uintptr_t)delta | (uintptr_t)weight | (uintptr_t)out) % 16 == 0,
               "mh_add_rms_norm: operands must be 16-byte aligned");
    hipLaunchKernelGGL(add_rms_norm_kernel, dim3(rows), dim3(256), 0, as_stream(stream), (half_t*)h, (const half_t*)delta,
                       (const half_t*)weight, (half_t*)out, hidden, eps);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

int mh_argmax(mh_stream_t stream, const void* logits, int32_t* out, int rows, int cols) {
    MH_REQUIRE(rows >= 0 && cols > 0, "mh_argmax: bad shape %d x %d", rows, cols);
    if (rows == 0) return MH_OK;
    MH_REQUIRE(logits && out, "mh_argmax: null pointer");
    hipLaunchKernelGGL(argmax_advance_kernel, dim3(rows), dim3(1024), 0, as_stream(stream), (const half_t*)logits, out,
                       (int32_t*)nullptr, (int32_t*)nullptr, (const int32_t*)nullptr, cols);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

int mh_rope_kv_append(mh_stream_t stream, const void* qkv, const float* freqs_cos, const float* freqs_sin,
                      const int32_t* positions, void* q_out, void* k_cache, void* vt_cache, int batch, int n_q_heads,
                      int n_kv_heads, int head_dim, int max_seq) {
    MH_REQUIRE(batch >= 0, "mh_rope_kv_append: bad batch %d", batch);
    if (batch == 0) return MH_OK;
    MH_REQUIRE(qkv && freqs_cos && freqs_sin && positions && q_out && k_cache && vt_cache,
               "mh_rope_kv_append: null pointer");
    MH_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && n_q_heads > 0 && n_kv_heads > 0, "mh_rope_kv_append: bad sizes");
    MH_REQUIRE(max_seq >= kVTile && max_seq % kVTile == 0, "mh_rope_kv_append: max_seq must be a multiple of 64, got %d",
               max_seq);
    hipLaunchKernelGGL(rope_kv_append_kernel, dim3(n_q_heads + 2 * n_kv_heads, batch), dim3(64), 0, as_stream(stream),
                       (const half_t*)qkv, freqs_cos, freqs_sin, positions, (half_t*)q_out, (half_t*)k_cache,
                       (half_t*)vt_cache, n_q_heads, n_kv_heads, head_dim, max_seq);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

int mh_llama_create(void** handle, const mh_llama_config* cfg) {
    MH_REQUIRE(handle && cfg, "mh_llama_create: null argument");
    MH_REQUIRE(cfg->n_layers > 0 && cfg->hidden > 0 && cfg->ffn > 0 && cfg->vocab > 0, "mh_llama_create: bad sizes");
    MH_REQUIRE(cfg->head_dim == 128, "mh_llama_create: head_dim must be 128, got %d", cfg->head_dim);
    MH_REQUIRE(cfg->n_kv_heads > 0 && cfg->n_q_heads % cfg->n_kv_heads == 0, "mh_llama_create: bad head counts");
    const int g = cfg->n_q_heads / cfg->n_kv_heads;
    MH_REQUIRE(g == 1 || g == 2 || g == 4 || g == 8, "mh_llama_create: %d query heads per KV head unsupported", g);
    MH_REQUIRE(cfg->max_seq >= kVTile && cfg->max_seq % kVTile == 0, "mh_llama_create: max_seq must be a multiple of 64, got %d",
               cfg->max_seq);
    MH_REQUIRE(cfg->hidden % 8 == 0 && cfg->hidden <= 8192, "mh_llama_create: hidden must be <= 8192 and a multiple of 8");
    MH_REQUIRE(cfg->ffn % 128 == 0, "mh_llama_create: ffn must be a multiple of 128 (gate/up interleave)");
    {
        const int rc = f16_gemv_prepare();  // the lm_head kernel's LDS attribute, ahead of any recording
        if (rc) return rc;
    }
    Llama* m = new (std::nothrow) Llama();
    MH_REQUIRE(m != nullptr, "mh_llama_create: out of host memory");
    m->cfg = *cfg;
    m->layers.resize(cfg->n_layers);
    memset(m->layers.data(), 0, sizeof(mh_llama_layer) * cfg->n_layers);
    *handle = m;
    return MH_OK;
}

int mh_llama_destroy(void* handle) {
    Llama* m = reinterpret_cast<Llama*>(handle);
    if (m) m->drop_graphs();
    delete m;
    return MH_OK;
}

int mh_llama_set_layer(void* handle, int layer, const mh_llama_layer* l) {
    Llama* m = reinterpret_cast<Llama*>(handle);
    MH_REQUIRE(m && l, "mh_llama_set_layer: null argument");
    MH_REQUIRE(layer >= 0 && layer < m->cfg.n_layers, "mh_llama_set_layer: layer %d out of range", layer);
    m->layers[layer] = *l;
    m->drop_graphs();  // recorded steps hold the old pointers
    return MH_OK;
}

int mh_llama_set_globals(void* handle, const void* embed, const void* lm_head, const void* final_norm,
                         const float* freqs_cos, const float* freqs_sin) {
    Llama* m = reinterpret_cast<Llama*>(handle);
    MH_REQUIRE(m && embed && lm_head && final_norm && freqs_cos && freqs_sin, "mh_llama_set_globals: null argument");
    m->embed = embed;
    m->lm_head = lm_head;
    m->final_norm = final_norm;
    m->cos = freqs_cos;
    m->sin = freqs_sin;
    m->drop_graphs();
    return MH_OK;
}

size_t mh_llama_scratch_bytes(void* handle, int batch) {
    Llama* m = reinterpret_cast<Llama*>(handle);
    if (!m || batch <= 0) return 0;
    return carve(*m, batch, nullptr).total;
}

int mh_llama_norm_clamped(void* handle, mh_stream_t stream, int batch, const void* scratch, int32_t* clamped) {
    Llama* m = reinterpret_cast<Llama*>(handle);
    MH_REQUIRE(m != nullptr && batch > 0 && scratch && clamped, "mh_llama_norm_clamped: bad argument");
    const Scratch s = carve(*m, batch, reinterpret_cast<char*>(const_cast<void*>(scratch)));
    unsigned word = 0;
    MH_CHECK_HIP(hipMemcpyAsync(&word, s.norm_clamped, sizeof(word), hipMemcpyDeviceToHost, as_stream(stream)));
    MH_CHECK_HIP(hipStreamSynchronize(as_stream(stream)));
    *clamped = word != 0;
    return MH_OK;
}

}  // extern "C"

// One decode step is the same sequence of launches on the same buffers for every
// token (the position and the token travel in device memory), so it can be
// recorded once into a HIP graph and replayed: `replay` does that, keeping the
// recorded step in the model for later calls on the same buffers.
static int decode_impl(void* handle, mh_stream_t stream, int batch, int32_t* tokens, int32_t* positions, int n_steps,
                       int32_t* out_tokens, void* logits_out, void* scratch, size_t scratch_bytes, bool replay) {
    Llama* m = reinterpret_cast<Llama*>(handle);
    MH_REQUIRE(m != nullptr, "mh_llama_decode: null handle");
    MH_REQUIRE(batch > 0 && n_steps >= 0, "mh_llama_decode: bad batch / steps");
    MH_REQUIRE(tokens && positions && scratch, "mh_llama_decode: null argument");
    MH_REQUIRE(m->embed != nullptr, "mh_llama_decode: globals not set");
    MH_REQUIRE((uintptr_t)scratch % 256 == 0, "mh_llama_decode: scratch must be 256-byte aligned");
    const Scratch s = carve(*m, batch, reinterpret_cast<char*>(scratch));
    if (scratch_bytes < s.total)
        return fail(MH_ERR_WORKSPACE, "mh_llama_decode: scratch of %zu bytes required, got %zu", s.total, scratch_bytes);
    const mh_llama_config& c = m->cfg;
    for (int l = 0; l < c.n_layers; ++l)
        MH_REQUIRE(m->layers[l].qkv.qweight && m->layers[l].k_cache, "mh_llama_decode: layer %d not set", l);
    hipStream_t st = as_stream(stream);
    const int qkv_n = (c.n_q_heads + 2 * c.n_kv_heads) * c.head_dim;
    const int g = c.n_q_heads / c.n_kv_heads;
    const int splits = attn_splits(*m, batch);
    const unsigned ew_grid = (unsigned)compute_units() * 4;
    const bool fused_silu = gemm_silu_pairs_supported(batch, 2 * c.ffn, c.hidden, c.group_size, c.bits);

    // activations of a linear whose rows were sorted by group at load time: gathered into that order
    auto ordered = [&](const half_t* x, const mh_qlinear& w, int k) -> const half_t* {
        if (w.perm == nullptr) return x;
        (void)mh_gather_columns(stream, x, w.perm, s.gathered, (size_t)batch, (size_t)k, MH_F16);
        return s.gathered;
    };
    auto linear = [&](const half_t* x, const mh_qlinear& w, half_t* y, int n, int k) -> int {
        x = ordered(x, w, k);
        if (w.bias != nullptr)
            return mh_gptq_linear(stream, x, w.qweight, w.qzeros, w.scales, nullptr, w.bias, y, batch, n, k,
                                  c.group_size, c.bits, s.gptq_ws, s.gptq_ws_bytes);
        return gptq_matmul_dispatch(st, x, w.qweight, w.qzeros, w.scales, y, batch, n, k, c.group_size, c.bits,
                                    s.gptq_ws, s.gptq_ws_bytes);
    };

    // The residual add and RMSNorm around the linears are folded into them where the
    // small-M product kernel serves the shapes: o and down add their result to the residual stream and leave per-tile
    // sums of squares, qkv and gate|up normalise that stream while staging it.
    const bool fused_norm =
        gemm_norm_fusion_supported(batch, c.hidden, c.n_q_heads * c.head_dim, c.group_size, c.bits, kEpilogueResidual) &&
        gemm_norm_fusion_supported(batch, c.hidden, c.ffn, c.group_size, c.bits, kEpilogueResidual) &&
        gemm_norm_fusion_supported(batch, qkv_n, c.hidden, c.group_size, c.bits, kEpilogueRopeAppend) &&
        gemm_norm_fusion_supported(batch, 2 * c.ffn, c.hidden, c.group_size, c.bits, kEpilogueSiluPairs) && fused_silu;
    // pieces the o and the down projection leave per row (they may run on different kernels)
    const int o_pieces = gemm_residual_ssq_pieces(batch, c.hidden, c.n_q_heads * c.head_dim, c.group_size, c.bits);
    const int down_pieces = gemm_residual_ssq_pieces(batch, c.hidden, c.ffn, c.group_size, c.bits);
    auto fused = [&](const half_t* x, const mh_qlinear& w, half_t* y, int n, int k, int epilogue,
                     SmallFuse fuse) -> int {
        fuse.bias = (const half_t*)w.bias;
        return gptq_matmul_fused(st, ordered(x, w, k), w.qweight, w.qzeros, w.scales, y, batch, n, k, c.group_size,
                                 c.bits, s.gptq_ws, s.gptq_ws_bytes, epilogue, fuse);
    };

    // every launch of one step; out_row / pos_base as for argmax_advance_kernel
    auto enqueue_step = [&](int32_t* out_row, const int32_t* pos_base) -> int {
        hipLaunchKernelGGL(embed_gather_kernel, dim3(batch), dim3(256), 0, st, tokens, (const half_t*)m->embed, s.h,
                           c.hidden, c.vocab);
        hipLaunchKernelGGL(add_rms_norm_kernel, dim3(batch), dim3(256), 0, st, s.h, (const half_t*)nullptr,
                           (const half_t*)m->layers[0].input_norm, s.xn, c.hidden, c.rms_eps);
        for (int l = 0; l < c.n_layers; ++l) {
            const mh_llama_layer& L = m->layers[l];
            int rc;
            if (fused_norm) {
                // RoPE and the cache append ride on the reduction of the q|k|v product
                SmallFuse f;
                f.rope_cos = m->cos;
                f.rope_sin = m->sin;
                f.positions = positions;
                f.q_out = s.q;
                f.k_cache = (half_t*)L.k_cache;
                f.vt_cache = (half_t*)L.v_cache;
                f.q_heads = c.n_q_heads;
                f.kv_heads = c.n_kv_heads;
                f.max_seq = c.max_seq;
                const half_t* x = s.xn;
                if (l > 0) {  // s.xn holds h * input_norm from the previous down projection
                    f.ssq_in = s.ssq_a;
                    f.ssq_tiles = down_pieces;
                    f.eps = c.rms_eps;
                }
                rc = fused(x, L.qkv, s.qkv, qkv_n, c.hidden, kEpilogueRopeAppend, f);
                if (rc) return rc;
            } else {
                rc = linear(s.xn, L.qkv, s.qkv, qkv_n, c.hidden);
                if (rc) return rc;
                hipLaunchKernelGGL(rope_kv_append_kernel, dim3(c.n_q_heads + 2 * c.n_kv_heads, batch), dim3(64), 0, st,
                                   s.qkv, m->cos, m->sin, positions, s.q, (half_t*)L.k_cache, (half_t*)L.v_cache,
                                   c.n_q_heads, c.n_kv_heads, c.head_dim, c.max_seq);
            }
            switch (g) {
                case 1: launch_attn<1>(st, *m, s, L, positions, batch, splits); break;
                case 2: launch_attn<2>(st, *m, s, L, positions, batch, splits); break;
                case 4: launch_attn<4>(st, *m, s, L, positions, batch, splits); break;
                default: launch_attn<8>(st, *m, s, L, positions, batch, splits); break;
            }
            if (fused_norm) {
                SmallFuse res;  // h += o; s.xn = h * post_norm
                res.ssq_out = s.ssq_b;
                res.next_norm_w = (const half_t*)L.post_norm;
                res.xw_out = s.xn;
                res.xw_clamped = s.norm_clamped;
                rc = fused(s.attn, L.o, s.h, c.hidden, c.n_q_heads * c.head_dim, kEpilogueResidual, res);
                if (rc) return rc;
                SmallFuse f;
                f.ssq_in = s.ssq_b;
                f.ssq_tiles = o_pieces;
                f.eps = c.rms_eps;
                rc = fused(s.xn, L.gate_up, s.act, 2 * c.ffn, c.hidden, kEpilogueSiluPairs, f);
                if (rc) return rc;
                res.ssq_out = s.ssq_a;  // h += down; s.xn = h * the next layer's input_norm
                res.next_norm_w = (const half_t*)(l + 1 < c.n_layers ? m->layers[l + 1].input_norm : m->final_norm);
                rc = fused(s.act, L.down, s.h, c.hidden, c.ffn, kEpilogueResidual, res);
                if (rc) return rc;
                continue;
            }
            rc = linear(s.attn, L.o, s.delta, c.hidden, c.n_q_heads * c.head_dim);
            if (rc) return rc;
            hipLaunchKernelGGL(add_rms_norm_kernel, dim3(batch), dim3(256), 0, st, s.h, s.delta,
                               (const half_t*)L.post_norm, s.xn, c.hidden, c.rms_eps);
            if (fused_silu) {
                rc = fused(s.xn, L.gate_up, s.act, 2 * c.ffn, c.hidden, kEpilogueSiluPairs, SmallFuse{});
                if (rc) return rc;
            } else {
                rc = linear(s.xn, L.gate_up, s.gu, 2 * c.ffn, c.hidden);
                if (rc) return rc;
                hipLaunchKernelGGL(silu_mul_fused_kernel, dim3(ew_grid), dim3(256), 0, st, s.gu, s.act, batch, c.ffn);
            }
            rc = linear(s.act, L.down, s.delta, c.hidden, c.ffn);
            if (rc) return rc;
            const half_t* next_norm =
                (const half_t*)(l + 1 < c.n_layers ? m->layers[l + 1].input_norm : m->final_norm);
            hipLaunchKernelGGL(add_rms_norm_kernel, dim3(batch), dim3(256), 0, st, s.h, s.delta, next_norm, s.xn,
                               c.hidden, c.rms_eps);
        }
        if (fused_norm)  // the last residual stream still wants its norm
            hipLaunchKernelGGL(add_rms_norm_kernel, dim3(batch), dim3(256), 0, st, s.h, (const half_t*)nullptr,
                               (const half_t*)m->final_norm, s.xn, c.hidden, c.rms_eps);
        int rc = mh_f16_matmul_nk(stream, s.xn, m->lm_head, s.logits, batch, c.vocab, c.hidden);
        if (rc) return rc;
        hipLaunchKernelGGL(argmax_advance_kernel, dim3(batch), dim3(1024), 0, st, s.logits, tokens, out_row, positions,
                           pos_base, c.vocab);
        MH_CHECK_LAUNCH();
        return MH_OK;
    };

    if (!replay) {
        for (int step = 0; step < n_steps; ++step) {
            const int rc = enqueue_step(out_tokens ? out_tokens + (size_t)step * batch : nullptr, nullptr);
            if (rc) return rc;
        }
    } else if (n_steps > 0) {
        MH_REQUIRE(st != nullptr, "mh_llama_decode_graph: needs a stream of its own (the null stream cannot record)");
        hipGraphExec_t exec = nullptr;
        for (const auto& g : m->graphs)
            if (g.batch == batch && g.tokens == tokens && g.positions == positions && g.out_tokens == out_tokens &&
                g.scratch == scratch)
                exec = g.exec;
        if (exec == nullptr) {
            MH_CHECK_HIP(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
            const int rc = enqueue_step(out_tokens, s.pos_base);
            hipGraph_t graph = nullptr;
            const hipError_t end = hipStreamEndCapture(st, &graph);  // also leaves capture mode after a failed step
            if (rc) {
                if (graph) (void)hipGraphDestroy(graph);
                return rc;
            }
            MH_CHECK_HIP(end);
            const hipError_t inst = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
            (void)hipGraphDestroy(graph);
            MH_CHECK_HIP(inst);
            m->graphs.push_back({batch, tokens, positions, out_tokens, scratch, exec});
        }
        // row r of the output belongs to the step that starts at pos_base + r
        MH_CHECK_HIP(hipMemcpyAsync(s.pos_base, positions, (size_t)batch * sizeof(int32_t), hipMemcpyDeviceToDevice, st));
        for (int step = 0; step < n_steps; ++step) MH_CHECK_HIP(hipGraphLaunch(exec, st));
    }
    if (logits_out && n_steps > 0)
        MH_CHECK_HIP(hipMemcpyAsync(logits_out, s.logits, (size_t)batch * c.vocab * 2, hipMemcpyDeviceToDevice, st));
    return MH_OK;
}

extern "C" {

int mh_llama_decode(void* handle, mh_stream_t stream, int batch, int32_t* tokens, int32_t* positions,
                    int n_steps, int32_t* out_tokens, void* logits_out, void* scratch, size_t scratch_bytes) {
    return decode_impl(handle, stream, batch, tokens, positions, n_steps, out_tokens, logits_out, scratch,
                       scratch_bytes, false);
}

int mh_llama_decode_graph(void* handle, mh_stream_t stream, int batch, int32_t* tokens, int32_t* positions,
                          int n_steps, int32_t* out_tokens, void* logits_out, void* scratch, size_t scratch_bytes) {
    return decode_impl(handle, stream, batch, tokens, positions, n_steps, out_tokens, logits_out, scratch,
                       scratch_bytes, true);
}

}  // extern "C"
