// RMSNorm, softmax (+ fused causal mask), row reductions, RoPE and SiLU*up.
//
// All of these are HBM-bound: one pass over the data where the row fits in
// registers, 16-byte loads, wave64 shuffle reductions (common.h).  A row belongs to
// 16, 64 or all 256 threads of a workgroup by its length (up to 128, 2048 or 3072,
// 8192 elements), so that short rows do not leave most of a workgroup idle; longer rows
// are walked twice by one workgroup, the second time out of the caches.  The view convention is
// the reference's: a tensor is seen as [a, b, c] and the operation runs along b
// (minit/cuda/dispatch.py:430-478).  c == 1 with 16-bit data takes the
// vectorised path; anything else takes the strided path.
#include "common.h"

namespace mh {

constexpr int kRowThreads = 256;
constexpr int kWideThreads = 1024;  // workgroup of the kernels for rows beyond the registers of kRowThreads threads
constexpr int kRowVec = 8;        // 16-bit elements per 16-byte load
constexpr int kRowMaxChunks = 4;  // register-resident rows: b <= 256 * 8 * 4 = 8192

template <typename T> struct Vec8 { uint4 raw; };

template <typename T>
__device__ __forceinline__ void unpack8(const uint4& raw, float* f) {
    const T* p = reinterpret_cast<const T*>(&raw);
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = Cvt<T>::to_f32(p[i]);
}

template <typename T>
__device__ __forceinline__ uint4 pack8(const float* f) {
    uint4 raw;
    T* p = reinterpret_cast<T*>(&raw);
#pragma unroll
    for (int i = 0; i < 8; ++i) p[i] = Cvt<T>::from_f32(f[i]);
    return raw;
}

// Sum / maximum over the LANES threads that share a row: the whole workgroup through LDS, or 16 / 64
// neighbouring lanes of a wave by shuffles.
template <int LANES>
__device__ __forceinline__ float group_sum(float v, float* smem) {
    if constexpr (LANES == kRowThreads) {
        return block_sum(v, smem);
    } else {
#pragma unroll
        for (int off = LANES / 2; off > 0; off >>= 1) v += __shfl_xor(v, off);
        return v;
    }
}
template <int LANES>
__device__ __forceinline__ float group_max(float v, float* smem) {
    if constexpr (LANES == kRowThreads) {
        return block_max(v, smem);
    } else {
#pragma unroll
        for (int off = LANES / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
        return v;
    }
}

// 16-byte accesses to data that is touched once: keep them from displacing what other
// workgroups reuse.
__device__ __forceinline__ uint4 stream_load(const uint4* p) {
    const uint4_t v = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(p));
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void stream_store(uint4* p, const uint4& v) {
    __builtin_nontemporal_store(uint4_t{v.x, v.y, v.z, v.w}, reinterpret_cast<uint4_t*>(p));
}

// ---- RMSNorm ------------------------------------------------------------------------------
// out = T( x / sqrt(sum(x^2)/b + eps) * w ), fp32 inside
// (minit/cuda/kernel/cuda/rms_norm.py:69-89).

template <typename T, int LANES, int CHUNKS>
__global__ __launch_bounds__(kRowThreads) void rms_norm_rows_kernel(
    const T* __restrict__ in, const T* __restrict__ weight, T* __restrict__ out, size_t a, size_t b, float eps) {
    __shared__ float smem[16];
    const size_t row = (size_t)blockIdx.x * (kRowThreads / LANES) + threadIdx.x / LANES;
    const int lane = threadIdx.x % LANES;
    if (LANES < kRowThreads && row >= a) return;  // whole groups of LANES threads
    const uint4* src = reinterpret_cast<const uint4*>(in + row * b);
    const uint4* wsrc = reinterpret_cast<const uint4*>(weight);
    uint4* dst = reinterpret_cast<uint4*>(out + row * b);
    const int nvec = (int)(b / kRowVec);
    uint4 regs[CHUNKS], wregs[CHUNKS];
    float ss = 0.f;
    // every load of the row and of the weight is requested before the first use; the row is read
    // once (streaming hint), the weight by every row (it stays cached)
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int v = c * LANES + lane;
        if (v < nvec) {
            regs[c] = stream_load(src + v);
            wregs[c] = wsrc[v];
        }
    }
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int v = c * LANES + lane;
        if (v < nvec) {
            float f[8];
            unpack8<T>(regs[c], f);
#pragma unroll
            for (int i = 0; i < 8; ++i) ss += f[i] * f[i];
        }
    }
    ss = group_sum<LANES>(ss, smem);
    const float rms = sqrtf(ss / (float)b + eps);
    // 16-bit storage: one division per row; x * (1 / rms) differs from x / rms by an fp32 ulp at most,
    // far below the storage type's step.  fp32 storage keeps the reference's x / rms * w.
    const float inv = 1.0f / rms;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int v = c * LANES + lane;
        if (v < nvec) {
            float f[8], w[8];
            unpack8<T>(regs[c], f);
            unpack8<T>(wregs[c], w);
#pragma unroll
            for (int i = 0; i < 8; ++i) f[i] = sizeof(T) == 2 ? f[i] * inv * w[i] : f[i] / rms * w[i];
            stream_store(dst + v, pack8<T>(f));
        }
    }
}

// Rows too long for the registers of a workgroup (more than 8192 elements): the row is walked twice with
// 16-byte loads, the second time out of the caches (plain loads first, streaming loads and stores last).
template <typename T>
__global__ __launch_bounds__(kWideThreads) void rms_norm_wide_kernel(
    const T* __restrict__ in, const T* __restrict__ weight, T* __restrict__ out, size_t b, float eps) {
    __shared__ float smem[16];
    const size_t row = blockIdx.x;
    const uint4* src = reinterpret_cast<const uint4*>(in + row * b);
    const uint4* wsrc = reinterpret_cast<const uint4*>(weight);
    uint4* dst = reinterpret_cast<uint4*>(out + row * b);
    const size_t nvec = b / kRowVec;
    float ss = 0.f;
#pragma unroll 4
    for (size_t v = threadIdx.x; v < nvec; v += kWideThreads) {
        float f[8];
        unpack8<T>(src[v], f);
#pragma unroll
        for (int i = 0; i < 8; ++i) ss += f[i] * f[i];
    }
    ss = block_sum(ss, smem);
    const float rms = sqrtf(ss / (float)b + eps);
    const float inv = 1.0f / rms;
#pragma unroll 4
    for (size_t v = threadIdx.x; v < nvec; v += kWideThreads) {
        float f[8], w[8];
        unpack8<T>(stream_load(src + v), f);
        unpack8<T>(wsrc[v], w);
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = sizeof(T) == 2 ? f[i] * inv * w[i] : f[i] / rms * w[i];
        stream_store(dst + v, pack8<T>(f));
    }
}

template <typename T>
__global__ __launch_bounds__(kRowThreads) void rms_norm_strided_kernel(
    const T* __restrict__ in, const T* __restrict__ weight, T* __restrict__ out,
    size_t a, size_t b, size_t c, float eps) {
    __shared__ float smem[16];
    const size_t lines = a * c;
    for (size_t line = blockIdx.x; line < lines; line += gridDim.x) {
        const size_t base = (line / c) * b * c + line % c;
        float ss = 0.f;
        for (size_t j = threadIdx.x; j < b; j += blockDim.x) {
            const float v = Cvt<T>::to_f32(in[base + j * c]);
            ss += v * v;
        }
        ss = block_sum(ss, smem);
        const float rms = sqrtf(ss / (float)b + eps);
        for (size_t j = threadIdx.x; j < b; j += blockDim.x) {
            const float v = Cvt<T>::to_f32(in[base + j * c]);
            out[base + j * c] = Cvt<T>::from_f32(v / rms * Cvt<T>::to_f32(weight[j]));
        }
    }
}

// ---- softmax --------------------------------------------------------------------------------
// p = exp(x - max) / sum(exp(x - max)), fp32 inside
// (minit/cuda/kernel/cuda/softmax.py:71-105).  The causal variant applies the
// models' scale and additive mask first (examples/llama3_70b.py:102-111): the
// scaled score is rounded to T as the separate divide kernel would, and
// positions j > offset + i contribute exp(-inf) = 0.

template <typename T, bool CAUSAL, int LANES, int CHUNKS>
__global__ __launch_bounds__(kRowThreads) void softmax_rows_kernel(
    const T* __restrict__ in, T* __restrict__ out, size_t a, size_t b, size_t s, size_t offset, float scale) {
    __shared__ float smem[16];
    const size_t row = (size_t)blockIdx.x * (kRowThreads / LANES) + threadIdx.x / LANES;
    const int lane = threadIdx.x % LANES;
    if (LANES < kRowThreads && row >= a) return;
    const uint4* src = reinterpret_cast<const uint4*>(in + row * b);
    uint4* dst = reinterpret_cast<uint4*>(out + row * b);
    const int nvec = (int)(b / kRowVec);
    const long limit = CAUSAL ? (long)(offset + row % s) : (long)b;  // last visible column
    float vals[CHUNKS][8];
    float mx = -INFINITY;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int v = c * LANES + lane;
        if (v < nvec) {
            const uint4 raw = stream_load(src + v);
            unpack8<T>(raw, vals[c]);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if (CAUSAL) {
                    float x = vals[c][i];
                    if (scale != 1.f) x = Cvt<T>::to_f32(Cvt<T>::from_f32(x * scale));
                    if ((long)v * 8 + i > limit) x = -INFINITY;
                    vals[c][i] = x;
                }
                mx = fmaxf(mx, vals[c][i]);
            }
        }
    }
    mx = group_max<LANES>(mx, smem);
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int v = c * LANES + lane;
        if (v < nvec) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                // 16-bit storage: exp(d) as 2^(d * log2 e) on the hardware's base-2 exponential (about an
                // fp32 ulp from expf, three orders below the storage step); fp32 storage keeps expf
                vals[c][i] = sizeof(T) == 2 ? __builtin_amdgcn_exp2f((vals[c][i] - mx) * 1.44269504088896340736f)
                                            : expf(vals[c][i] - mx);
                sum += vals[c][i];
            }
        }
    }
    sum = group_sum<LANES>(sum, smem);
    const float inv = 1.0f / sum;  // one division per row for 16-bit storage
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int v = c * LANES + lane;
        if (v < nvec) {
#pragma unroll
            for (int i = 0; i < 8; ++i) vals[c][i] = sizeof(T) == 2 ? vals[c][i] * inv : vals[c][i] / sum;
            stream_store(dst + v, pack8<T>(vals[c]));
        }
    }
}

// Rows of more than 8192 elements: maximum, sum and store in three walks over the row with 16-byte loads, the
// second and third out of the caches; the arithmetic of softmax_rows_kernel.
template <typename T, bool CAUSAL>
__global__ __launch_bounds__(kWideThreads) void softmax_wide_kernel(
    const T* __restrict__ in, T* __restrict__ out, size_t b, size_t s, size_t offset, float scale) {
    __shared__ float smem[16];
    const size_t row = blockIdx.x;
    const uint4* src = reinterpret_cast<const uint4*>(in + row * b);
    uint4* dst = reinterpret_cast<uint4*>(out + row * b);
    const size_t nvec = b / kRowVec;
    const long limit = CAUSAL ? (long)(offset + row % s) : (long)b;
    auto fetch = [&](size_t v, bool last, float* x) {
        unpack8<T>(last ? stream_load(src + v) : src[v], x);
        if (CAUSAL) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if (scale != 1.f) x[i] = Cvt<T>::to_f32(Cvt<T>::from_f32(x[i] * scale));
                if ((long)v * 8 + i > limit) x[i] = -INFINITY;
            }
        }
    };
    auto expd = [](float d) { return sizeof(T) == 2 ? __builtin_amdgcn_exp2f(d * 1.44269504088896340736f) : expf(d); };
    float mx = -INFINITY;
#pragma unroll 4
    for (size_t v = threadIdx.x; v < nvec; v += kWideThreads) {
        float x[8];
        fetch(v, false, x);
#pragma unroll
        for (int i = 0; i < 8; ++i) mx = fmaxf(mx, x[i]);
    }
    mx = block_max(mx, smem);
    float sum = 0.f;
#pragma unroll 4
    for (size_t v = threadIdx.x; v < nvec; v += kWideThreads) {
        float x[8];
        fetch(v, false, x);
#pragma unroll
        for (int i = 0; i < 8; ++i) sum += expd(x[i] - mx);
    }
    sum = block_sum(sum, smem);
    const float inv = 1.0f / sum;
#pragma unroll 4
    for (size_t v = threadIdx.x; v < nvec; v += kWideThreads) {
        float x[8];
        fetch(v, true, x);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = sizeof(T) == 2 ? expd(x[i] - mx) * inv : expd(x[i] - mx) / sum;
        stream_store(dst + v, pack8<T>(x));
    }
}

template <typename T, bool CAUSAL>
__global__ __launch_bounds__(kRowThreads) void softmax_strided_kernel(
    const T* __restrict__ in, T* __restrict__ out, size_t a, size_t b, size_t c, size_t s, size_t offset,
    float scale) {
    __shared__ float smem[16];
    const size_t lines = a * c;
    for (size_t line = blockIdx.x; line < lines; line += gridDim.x) {
        const size_t base = (line / c) * b * c + line % c;
        const long limit = CAUSAL ? (long)(offset + line % s) : (long)b;
        auto fetch = [&](size_t j) {
            float x = Cvt<T>::to_f32(in[base + j * c]);
            if (CAUSAL) {
                if (scale != 1.f) x = Cvt<T>::to_f32(Cvt<T>::from_f32(x * scale));
                if ((long)j > limit) x = -INFINITY;
            }
            return x;
        };
        float mx = -INFINITY;
        for (size_t j = threadIdx.x; j < b; j += blockDim.x) mx = fmaxf(mx, fetch(j));
        mx = block_max(mx, smem);
        float sum = 0.f;
        for (size_t j = threadIdx.x; j < b; j += blockDim.x) sum += expf(fetch(j) - mx);
        sum = block_sum(sum, smem);
        for (size_t j = threadIdx.x; j < b; j += blockDim.x)
            out[base + j * c] = Cvt<T>::from_f32(expf(fetch(j) - mx) / sum);
    }
}

// ---- reductions -------------------------------------------------------------------------------
// [a, b, c] -> [a, 1, c], fp32 accumulate, cast at the store
// (minit/cuda/kernel/cuda/reduce.py:76-92).

// MEAN: the sum is rounded to T and divided by T(b), rounded again, which is what the
// reference's mean composes (minit/functional/reduce.py:14-18: sum, fill, divide).
template <typename T>
__device__ __forceinline__ T mean_of_sum(float sum, size_t b) {
    const float s = Cvt<T>::to_f32(Cvt<T>::from_f32(sum));
    const float n = Cvt<T>::to_f32(Cvt<T>::from_f32((float)b));
    return Cvt<T>::from_f32(s / n);
}

template <typename T, bool IS_MAX, bool MEAN, int LANES>
__global__ __launch_bounds__(kRowThreads) void reduce_rows_kernel(const T* __restrict__ in,
                                                                 T* __restrict__ out, size_t a, size_t b) {
    __shared__ float smem[16];
    const size_t row = (size_t)blockIdx.x * (kRowThreads / LANES) + threadIdx.x / LANES;
    const int lane = threadIdx.x % LANES;
    if (LANES < kRowThreads && row >= a) return;
    const T* src = in + row * b;
    float acc = IS_MAX ? -INFINITY : 0.f;
    const size_t nvec = (sizeof(T) == 2 && (uintptr_t)src % 16 == 0) ? b / kRowVec : 0;
    const uint4* vsrc = reinterpret_cast<const uint4*>(src);
    for (size_t v = lane; v < nvec; v += LANES) {
        float f[8];
        const uint4 raw = vsrc[v];
        unpack8<T>(raw, f);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc = IS_MAX ? fmaxf(acc, f[i]) : acc + f[i];
    }
    for (size_t j = nvec * kRowVec + lane; j < b; j += LANES) {
        const float f = Cvt<T>::to_f32(src[j]);
        acc = IS_MAX ? fmaxf(acc, f) : acc + f;
    }
    acc = IS_MAX ? group_max<LANES>(acc, smem) : group_sum<LANES>(acc, smem);
    if (lane == 0) out[row] = MEAN ? mean_of_sum<T>(acc, b) : Cvt<T>::from_f32(acc);
}

// Long rows: the same walk by a workgroup of 1024 threads with streaming loads.  Sums over rows of 16384 /
// 28672 / 131072 / 1048576 elements: 5.9 / 7.0 / 6.9 / 6.9 TB/s against 6.15 / 6.0 / 5.8 / 2.1 on 256 threads,
// so rows of 24576 elements and more come here.
constexpr size_t kReduceWideMin = 24576;
template <typename T, bool IS_MAX, bool MEAN>
__global__ __launch_bounds__(kWideThreads) void reduce_wide_kernel(const T* __restrict__ in, T* __restrict__ out, size_t b) {
    __shared__ float smem[16];
    const size_t row = blockIdx.x;
    const T* src = in + row * b;
    float acc = IS_MAX ? -INFINITY : 0.f;
    const size_t nvec = (sizeof(T) == 2 && (uintptr_t)src % 16 == 0) ? b / kRowVec : 0;
    const uint4* vsrc = reinterpret_cast<const uint4*>(src);
#pragma unroll 4
    for (size_t v = threadIdx.x; v < nvec; v += kWideThreads) {
        float f[8];
        unpack8<T>(stream_load(vsrc + v), f);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc = IS_MAX ? fmaxf(acc, f[i]) : acc + f[i];
    }
    for (size_t j = nvec * kRowVec + threadIdx.x; j < b; j += kWideThreads) {
        const float f = Cvt<T>::to_f32(src[j]);
        acc = IS_MAX ? fmaxf(acc, f) : acc + f;
    }
    acc = IS_MAX ? block_max(acc, smem) : block_sum(acc, smem);
    if (threadIdx.x == 0) out[row] = MEAN ? mean_of_sum<T>(acc, b) : Cvt<T>::from_f32(acc);
}

// c > 1: one thread per output element, coalesced across c.
template <typename T, bool IS_MAX, bool MEAN = false>
__global__ void reduce_strided_kernel(const T* __restrict__ in, T* __restrict__ out, size_t a, size_t b,
                                      size_t c) {
    const size_t total = a * c;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
        const size_t base = (idx / c) * b * c + idx % c;
        float acc = IS_MAX ? -INFINITY : 0.f;
        for (size_t j = 0; j < b; ++j) {
            const float f = Cvt<T>::to_f32(in[base + j * c]);
            acc = IS_MAX ? fmaxf(acc, f) : acc + f;
        }
        out[idx] = MEAN ? mean_of_sum<T>(acc, b) : Cvt<T>::from_f32(acc);
    }
}

// ---- RoPE ----------------------------------------------------------------------------------------
// o[2i] = x[2i] c - x[2i+1] s ; o[2i+1] = x[2i+1] c + x[2i] s, fp32 math, one
// rounding (minit/cuda/kernel/cuda/rope.py:58-73).  One thread per complex pair.

template <typename T>
__global__ void rope_kernel(const T* __restrict__ in, const float* __restrict__ freqs_cos,
                            const float* __restrict__ freqs_sin, const int32_t* __restrict__ positions,
                            T* __restrict__ out, size_t bs, size_t seq, size_t nh, size_t half) {
    const size_t total = bs * seq * nh * half;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
        const size_t i = idx % half;
        const size_t bsq = idx / (half * nh);  // b * seq + s
        const size_t pos = positions ? (size_t)positions[bsq] : bsq % seq;
        const float c = freqs_cos[pos * half + i], s = freqs_sin[pos * half + i];
        const float re = Cvt<T>::to_f32(in[idx * 2]), im = Cvt<T>::to_f32(in[idx * 2 + 1]);
        out[idx * 2] = Cvt<T>::from_f32(re * c - im * s);
        out[idx * 2 + 1] = Cvt<T>::from_f32(im * c + re * s);
    }
}

// 16-bit fast path: one thread per four pairs (16 bytes of x, 16 bytes of each table).
template <typename T>
__global__ void rope_vec_kernel(const T* __restrict__ in, const float* __restrict__ freqs_cos,
                                const float* __restrict__ freqs_sin, const int32_t* __restrict__ positions,
                                T* __restrict__ out, size_t bs, size_t seq, size_t nh, size_t half) {
    const size_t quads = half / 4;
    const size_t total = bs * seq * nh * quads;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
        const size_t qd = idx % quads;
        const size_t bsq = idx / (quads * nh);
        const size_t pos = positions ? (size_t)positions[bsq] : bsq % seq;
        const float4 c = *reinterpret_cast<const float4*>(freqs_cos + pos * half + qd * 4);
        const float4 s = *reinterpret_cast<const float4*>(freqs_sin + pos * half + qd * 4);
        const uint4 raw = stream_load(reinterpret_cast<const uint4*>(in) + idx);  // x is touched once, the tables by every head
        float f[8], o[8];
        unpack8<T>(raw, f);
        const float cs[4] = {c.x, c.y, c.z, c.w}, sn[4] = {s.x, s.y, s.z, s.w};
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            o[2 * p] = f[2 * p] * cs[p] - f[2 * p + 1] * sn[p];
            o[2 * p + 1] = f[2 * p + 1] * cs[p] + f[2 * p] * sn[p];
        }
        stream_store(reinterpret_cast<uint4*>(out) + idx, pack8<T>(o));
    }
}

// ---- SiLU(gate) * up ---------------------------------------------------------------------------------
// EXACT reproduces the three launches of the reference (sigmoid rounded to T,
// T multiply, T multiply: minit/cuda/dispatch.py:137,143); otherwise fp32 until
// the store.

template <typename T, bool EXACT>
__device__ __forceinline__ float silu_mul_one(float g, float u) {
    if (EXACT) {
        const float sig = Cvt<T>::to_f32(Cvt<T>::from_f32((float)(1.0 / (1.0 + (double)expf(-g)))));
        const float a = Cvt<T>::to_f32(Cvt<T>::from_f32(g * sig));
        return a * u;
    }
    return g / (1.f + expf(-g)) * u;
}

template <typename T, bool EXACT>
__global__ void silu_mul_kernel(const T* __restrict__ gate, const T* __restrict__ up, T* __restrict__ out,
                                size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const bool aligned = (((uintptr_t)gate | (uintptr_t)up | (uintptr_t)out) % 16 == 0) && sizeof(T) == 2;
    const size_t nvec = aligned ? n / 8 : 0;
    for (size_t v = (size_t)blockIdx.x * blockDim.x + threadIdx.x; v < nvec; v += stride) {
        float g[8], u[8];
        const uint4 graw = reinterpret_cast<const uint4*>(gate)[v];
        const uint4 uraw = reinterpret_cast<const uint4*>(up)[v];
        unpack8<T>(graw, g);
        unpack8<T>(uraw, u);
#pragma unroll
        for (int i = 0; i < 8; ++i) g[i] = silu_mul_one<T, EXACT>(g[i], u[i]);
        reinterpret_cast<uint4*>(out)[v] = pack8<T>(g);
    }
    for (size_t j = nvec * 8 + (size_t)blockIdx.x * blockDim.x + threadIdx.x; j < n; j += stride)
        out[j] = Cvt<T>::from_f32(silu_mul_one<T, EXACT>(Cvt<T>::to_f32(gate[j]), Cvt<T>::to_f32(up[j])));
}

// The two element-wise kernels the models' silu uses on its own (examples/llama3_70b.py:
// 44-45): sigmoid with the reference's expression, 1.0 / (1.0 + expf((float)-x)) in
// double and one rounding (minit/cuda/dispatch.py:143), and the product in T (:137).
// OP 0: sigmoid(a); OP 1: a * b; OP 2: a + b (the residual add, `{0} + {1}`, :135).
template <typename T, int OP>
__device__ __forceinline__ float elementwise_one(float a, float b) {
    if (OP == 0) return (float)(1.0 / (1.0 + (double)expf(-a)));  // double -> float -> T rounds like double -> T: 24 >= 2 * 11 + 2
    if (OP == 2) return a + b;  // fp32 sum of two 16-bit values, rounded to T at the store: the result of a half add
    return a * b;
}

template <typename T, int OP>
__global__ void elementwise_kernel(const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ out, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const bool aligned = (((uintptr_t)a | (uintptr_t)b | (uintptr_t)out) % 16 == 0) && sizeof(T) == 2;
    const size_t nvec = aligned ? n / 8 : 0;
    for (size_t v = (size_t)blockIdx.x * blockDim.x + threadIdx.x; v < nvec; v += stride) {
        float x[8], y[8];
        unpack8<T>(reinterpret_cast<const uint4*>(a)[v], x);
        if (OP != 0) unpack8<T>(reinterpret_cast<const uint4*>(b)[v], y);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = elementwise_one<T, OP>(x[i], OP != 0 ? y[i] : 0.f);
        reinterpret_cast<uint4*>(out)[v] = pack8<T>(x);
    }
    for (size_t j = nvec * 8 + (size_t)blockIdx.x * blockDim.x + threadIdx.x; j < n; j += stride)
        out[j] = Cvt<T>::from_f32(elementwise_one<T, OP>(Cvt<T>::to_f32(a[j]), OP != 0 ? Cvt<T>::to_f32(b[j]) : 0.f));
}

static unsigned grid_for(size_t work_items, int per_block) {
    size_t blocks = (work_items + per_block - 1) / per_block;
    const size_t cap = (size_t)compute_units() * 16;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return (unsigned)blocks;
}

// Contiguous rows of 16-bit elements in whole 16-byte pieces: the vectorised kernels.
static bool rows_vector_path(const void* in, const void* out, size_t b, size_t c, size_t elem) {
    return c == 1 && elem == 2 && b % kRowVec == 0 && ((uintptr_t)in | (uintptr_t)out) % 16 == 0;
}
static bool rows_fit_registers(size_t b) { return b <= (size_t)kRowThreads * kRowVec * kRowMaxChunks; }
// Threads per row: 16 up to 128 elements, 64 up to `most64` (2048 for RMSNorm, whose lanes hold the weight's
// pieces as well, 3072 for softmax and the reductions: softmax over 2056 / 3072 / 4096 elements on 64 threads
// 5.7 / 6.3 / 6.2 TB/s, on 256 threads 4.8 / 6.0 / 6.5; RMSNorm 4.5 / 5.4 / 5.4 against 4.3 / 5.7 / 6.4), else
// the workgroup.
static int rows_lanes(size_t b, size_t most64) { return b <= 16 * kRowVec ? 16 : b <= most64 ? 64 : kRowThreads; }
static unsigned rows_grid(size_t a, int lanes) {
    const size_t per = kRowThreads / lanes;
    return (unsigned)((a + per - 1) / per);
}

template <typename T>
static int rms_norm_t(hipStream_t st, const void* in, const void* weight, void* out, size_t a, size_t b,
                      size_t c, float eps) {
    if (rows_vector_path(in, out, b, c, sizeof(T)) && (uintptr_t)weight % 16 == 0) {
        const int lanes = rows_lanes(b, 2048);
#define MH_RMS_ROWS(LANES, CHUNKS)                                                                                   \
    hipLaunchKernelGGL((rms_norm_rows_kernel<T, LANES, CHUNKS>), dim3(rows_grid(a, LANES)), dim3(kRowThreads), 0, st,    \
                       (const T*)in, (const T*)weight, (T*)out, a, b, eps)
        if (!rows_fit_registers(b))
            hipLaunchKernelGGL(rms_norm_wide_kernel<T>, dim3((unsigned)a), dim3(kWideThreads), 0, st, (const T*)in,
                               (const T*)weight, (T*)out, b, eps);
        else if (lanes == 16)
            MH_RMS_ROWS(16, 1);
        else if (lanes == 64)
            MH_RMS_ROWS(64, 4);
        else
            MH_RMS_ROWS(kRowThreads, kRowMaxChunks);
#undef MH_RMS_ROWS
    } else {
        hipLaunchKernelGGL(rms_norm_strided_kernel<T>, dim3(grid_for(a * c, 1)), dim3(kRowThreads), 0, st,
                           (const T*)in, (const T*)weight, (T*)out, a, b, c, eps);
    }
    MH_CHECK_LAUNCH();
    return MH_OK;
}

template <typename T, bool CAUSAL>
static int softmax_t(hipStream_t st, const void* in, void* out, size_t a, size_t b, size_t c, size_t s,
                     size_t offset, float scale) {
    if (rows_vector_path(in, out, b, c, sizeof(T))) {
        const int lanes = rows_lanes(b, 3072);
#define MH_SOFTMAX_ROWS(LANES, CHUNKS)                                                                               \
    hipLaunchKernelGGL((softmax_rows_kernel<T, CAUSAL, LANES, CHUNKS>), dim3(rows_grid(a, LANES)), dim3(kRowThreads), 0, \
                       st, (const T*)in, (T*)out, a, b, s, offset, scale)
        if (!rows_fit_registers(b))
            hipLaunchKernelGGL((softmax_wide_kernel<T, CAUSAL>), dim3((unsigned)a), dim3(kWideThreads), 0, st,
                               (const T*)in, (T*)out, b, s, offset, scale);
        else if (lanes == 16)
            MH_SOFTMAX_ROWS(16, 1);
        else if (lanes == 64 && b <= 64 * kRowVec * 4)
            MH_SOFTMAX_ROWS(64, 4);
        else if (lanes == 64)
            MH_SOFTMAX_ROWS(64, 8);
        else
            MH_SOFTMAX_ROWS(kRowThreads, kRowMaxChunks);
#undef MH_SOFTMAX_ROWS
    } else {
        hipLaunchKernelGGL((softmax_strided_kernel<T, CAUSAL>), dim3(grid_for(a * c, 1)), dim3(kRowThreads), 0,
                           st, (const T*)in, (T*)out, a, b, c, s, offset, scale);
    }
    MH_CHECK_LAUNCH();
    return MH_OK;
}

template <typename T, bool IS_MAX, bool MEAN = false>
static int reduce_t(hipStream_t st, const void* in, void* out, size_t a, size_t b, size_t c) {
    if (c == 1) {
        const int lanes = rows_lanes(b, 3072);
#define MH_REDUCE_ROWS(LANES)                                                                                        \
    hipLaunchKernelGGL((reduce_rows_kernel<T, IS_MAX, MEAN, LANES>), dim3(rows_grid(a, LANES)), dim3(kRowThreads), 0, \
                       st, (const T*)in, (T*)out, a, b)
        if (b >= kReduceWideMin)
            hipLaunchKernelGGL((reduce_wide_kernel<T, IS_MAX, MEAN>), dim3((unsigned)a), dim3(kWideThreads), 0, st,
                               (const T*)in, (T*)out, b);
        else if (lanes == 16)
            MH_REDUCE_ROWS(16);
        else if (lanes == 64)
            MH_REDUCE_ROWS(64);
        else
            MH_REDUCE_ROWS(kRowThreads);
#undef MH_REDUCE_ROWS
    } else {
        hipLaunchKernelGGL((reduce_strided_kernel<T, IS_MAX, MEAN>), dim3(grid_for(a * c, 256)), dim3(256), 0, st,
                           (const T*)in, (T*)out, a, b, c);
    }
    MH_CHECK_LAUNCH();
    return MH_OK;
}

}  // namespace mh

using namespace mh;

// x[r, c] = T(x[r, c] + bias[c]) in place: the broadcast add that follows the
// quantized product in a linear with bias (examples/qwen1_5_int8.py:311-317), one
// rounding in the storage type like the reference's element-wise Add.
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ x, const T* __restrict__ bias, size_t rows, size_t cols) {
    const size_t n = rows * cols;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const T sum = Cvt<T>::from_f32(Cvt<T>::to_f32(x[i]) + Cvt<T>::to_f32(bias[i % cols]));
        x[i] = sum;
    }
}

// out[r, j] = x[r, index[j]]: the activations in the row order of a weight that was
// sorted by group at load time.  An index outside [0, cols) is clamped.
template <typename T>
__global__ void gather_columns_kernel(const T* __restrict__ x, const int32_t* __restrict__ index, T* __restrict__ out,
                                      size_t rows, size_t cols) {
    const size_t n = rows * cols;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / cols, j = i % cols;
        const int src = min(max(index[j], 0), (int)cols - 1);
        out[i] = x[r * cols + src];
    }
}

#define MH_DISPATCH_DTYPE(dtype, who, CALL)                                         \
    switch (dtype) {                                                                \
        case MH_F16: { typedef half_t T; CALL; }                                    \
        case MH_BF16: { typedef __hip_bfloat16 T; CALL; }                           \
        case MH_F32: { typedef float T; CALL; }                                     \
        default: return fail(MH_ERR_INVALID, who ": unknown dtype %d", dtype);      \
    }

extern "C" {

int mh_rms_norm(mh_stream_t stream, const void* in, const void* weight, void* out, size_t a, size_t b,
                size_t c, double eps, int dtype) {
    if (a * b * c == 0) return MH_OK;
    MH_REQUIRE(in && weight && out, "mh_rms_norm: null pointer");
    MH_REQUIRE(a <= 0x7fffffffu, "mh_rms_norm: too many rows");
    MH_DISPATCH_DTYPE(dtype, "mh_rms_norm",
                      return rms_norm_t<T>(as_stream(stream), in, weight, out, a, b, c, (float)eps));
}

int mh_softmax(mh_stream_t stream, const void* in, void* out, size_t a, size_t b, size_t c, int dtype) {
    if (a * b * c == 0) return MH_OK;
    MH_REQUIRE(in && out, "mh_softmax: null pointer");
    MH_REQUIRE(a <= 0x7fffffffu, "mh_softmax: too many rows");
    MH_DISPATCH_DTYPE(dtype, "mh_softmax",
                      return (softmax_t<T, false>(as_stream(stream), in, out, a, b, c, 1, 0, 1.f)));
}

int mh_softmax_causal(mh_stream_t stream, const void* in, void* out, size_t rows_outer, size_t s, size_t t,
                      size_t offset, float scale, int dtype) {
    if (rows_outer * s * t == 0) return MH_OK;
    MH_REQUIRE(in && out, "mh_softmax_causal: null pointer");
    MH_REQUIRE(t == offset + s, "mh_softmax_causal: t=%zu must equal offset=%zu + s=%zu", t, offset, s);
    MH_REQUIRE(rows_outer * s <= 0x7fffffffu, "mh_softmax_causal: too many rows");
    MH_DISPATCH_DTYPE(dtype, "mh_softmax_causal",
                      return (softmax_t<T, true>(as_stream(stream), in, out, rows_outer * s, t, 1, s, offset, scale)));
}

int mh_sum(mh_stream_t stream, const void* in, void* out, size_t a, size_t b, size_t c, int dtype) {
    if (a * c == 0) return MH_OK;
    MH_REQUIRE(in && out, "mh_sum: null pointer");
    MH_REQUIRE(a <= 0x7fffffffu, "mh_sum: too many rows");
    MH_DISPATCH_DTYPE(dtype, "mh_sum", return (reduce_t<T, false>(as_stream(stream), in, out, a, b, c)));
}

int mh_max(mh_stream_t stream, const void* in, void* out, size_t a, size_t b, size_t c, int dtype) {
    if (a * c == 0) return MH_OK;
    MH_REQUIRE(in && out, "mh_max: null pointer");
    MH_REQUIRE(a <= 0x7fffffffu, "mh_max: too many rows");
    MH_DISPATCH_DTYPE(dtype, "mh_max", return (reduce_t<T, true>(as_stream(stream), in, out, a, b, c)));
}

int mh_mean(mh_stream_t stream, const void* in, void* out, size_t a, size_t b, size_t c, int dtype) {
    if (a * c == 0) return MH_OK;
    MH_REQUIRE(in && out, "mh_mean: null pointer");
    MH_REQUIRE(b > 0, "mh_mean: empty axis");
    MH_REQUIRE(a <= 0x7fffffffu, "mh_mean: too many rows");
    MH_DISPATCH_DTYPE(dtype, "mh_mean", return (reduce_t<T, false, true>(as_stream(stream), in, out, a, b, c)));
}

int mh_rope(mh_stream_t stream, const void* in, const float* freqs_cos, const float* freqs_sin,
            const int32_t* positions, void* out, size_t bs, size_t seq, size_t nh, size_t hs, int dtype) {
    if (bs * seq * nh * hs == 0) return MH_OK;
    MH_REQUIRE(in && out && freqs_cos && freqs_sin, "mh_rope: null pointer");
    MH_REQUIRE(hs % 2 == 0, "mh_rope: head size %zu must be even", hs);
    const size_t half = hs / 2;
    hipStream_t st = as_stream(stream);
    const bool vec = dtype != MH_F32 && half % 4 == 0 &&
                     (((uintptr_t)in | (uintptr_t)out | (uintptr_t)freqs_cos | (uintptr_t)freqs_sin) % 16 == 0);
    const size_t items = bs * seq * nh * (vec ? half / 4 : half);
    const unsigned grid = grid_for(items, 256);
#define MH_ROPE_CALL                                                                                         \
    if (vec)                                                                                                 \
        hipLaunchKernelGGL(rope_vec_kernel<T>, dim3(grid), dim3(256), 0, st, (const T*)in, freqs_cos,        \
                           freqs_sin, positions, (T*)out, bs, seq, nh, half);                                \
    else                                                                                                     \
        hipLaunchKernelGGL(rope_kernel<T>, dim3(grid), dim3(256), 0, st, (const T*)in, freqs_cos, freqs_sin, \
                           positions, (T*)out, bs, seq, nh, half);                                           \
    MH_CHECK_LAUNCH();                                                                                       \
    return MH_OK;
    MH_DISPATCH_DTYPE(dtype, "mh_rope", MH_ROPE_CALL);
#undef MH_ROPE_CALL
}

int mh_silu_mul(mh_stream_t stream, const void* gate, const void* up, void* out, size_t n, int exact,
                int dtype) {
    if (n == 0) return MH_OK;
    MH_REQUIRE(gate && up && out, "mh_silu_mul: null pointer");
    hipStream_t st = as_stream(stream);
    const unsigned grid = grid_for(n / 8 + 1, 256);
#define MH_SILU_CALL                                                                                  \
    if (exact)                                                                                        \
        hipLaunchKernelGGL((silu_mul_kernel<T, true>), dim3(grid), dim3(256), 0, st, (const T*)gate,  \
                           (const T*)up, (T*)out, n);                                                 \
    else                                                                                              \
        hipLaunchKernelGGL((silu_mul_kernel<T, false>), dim3(grid), dim3(256), 0, st, (const T*)gate, \
                           (const T*)up, (T*)out, n);                                                 \
    MH_CHECK_LAUNCH();                                                                                \
    return MH_OK;
    MH_DISPATCH_DTYPE(dtype, "mh_silu_mul", MH_SILU_CALL);
#undef MH_SILU_CALL
}

int mh_gather_columns(mh_stream_t stream, const void* x, const int32_t* index, void* out, size_t rows, size_t cols,
                      int dtype) {
    if (rows * cols == 0) return MH_OK;
    MH_REQUIRE(x && index && out, "mh_gather_columns: null pointer");
    MH_REQUIRE(x != out, "mh_gather_columns: not in place");
    MH_REQUIRE(cols <= 0x7fffffffu, "mh_gather_columns: too many columns");
    const unsigned grid = grid_for(rows * cols, 256);
#define MH_GATHER_CALL                                                                                          \
    hipLaunchKernelGGL(gather_columns_kernel<T>, dim3(grid), dim3(256), 0, as_stream(stream), (const T*)x, index, \
                       (T*)out, rows, cols);                                                                    \
    MH_CHECK_LAUNCH();                                                                                          \
    return MH_OK;
    MH_DISPATCH_DTYPE(dtype, "mh_gather_columns", MH_GATHER_CALL);
#undef MH_GATHER_CALL
}

int mh_sigmoid(mh_stream_t stream, const void* in, void* out, size_t n, int dtype) {
    if (n == 0) return MH_OK;
    MH_REQUIRE(in && out, "mh_sigmoid: null pointer");
    const unsigned grid = grid_for(n / 8 + 1, 256);
#define MH_EW_CALL                                                                                           \
    hipLaunchKernelGGL((elementwise_kernel<T, 0>), dim3(grid), dim3(256), 0, as_stream(stream), (const T*)in, \
                       (const T*)in, (T*)out, n);                                                            \
    MH_CHECK_LAUNCH();                                                                                       \
    return MH_OK;
    MH_DISPATCH_DTYPE(dtype, "mh_sigmoid", MH_EW_CALL);
#undef MH_EW_CALL
}

int mh_add(mh_stream_t stream, const void* a, const void* b, void* out, size_t n, int dtype) {
    if (n == 0) return MH_OK;
    MH_REQUIRE(a && b && out, "mh_add: null pointer");
    const unsigned grid = grid_for(n / 8 + 1, 256);
#define MH_EW_CALL                                                                                          \
    hipLaunchKernelGGL((elementwise_kernel<T, 2>), dim3(grid), dim3(256), 0, as_stream(stream), (const T*)a, \
                       (const T*)b, (T*)out, n);                                                            \
    MH_CHECK_LAUNCH();                                                                                      \
    return MH_OK;
    MH_DISPATCH_DTYPE(dtype, "mh_add", MH_EW_CALL);
#undef MH_EW_CALL
}

int mh_multiply(mh_stream_t stream, const void* a, const void* b, void* out, size_t n, int dtype) {
    if (n == 0) return MH_OK;
    MH_REQUIRE(a && b && out, "mh_multiply: null pointer");
    const unsigned grid = grid_for(n / 8 + 1, 256);
#define MH_EW_CALL                                                                                          \
    hipLaunchKernelGGL((elementwise_kernel<T, 1>), dim3(grid), dim3(256), 0, as_stream(stream), (const T*)a, \
                       (const T*)b, (T*)out, n);                                                            \
    MH_CHECK_LAUNCH();                                                                                      \
    return MH_OK;
    MH_DISPATCH_DTYPE(dtype, "mh_multiply", MH_EW_CALL);
#undef MH_EW_CALL
}

int mh_add_bias(mh_stream_t stream, void* x, const void* bias, size_t rows, size_t cols, int dtype) {
    if (rows * cols == 0) return MH_OK;
    MH_REQUIRE(x && bias, "mh_add_bias: null pointer");
    hipStream_t st = as_stream(stream);
    const unsigned grid = grid_for(rows * cols, 256);
#define MH_BIAS_CALL                                                                                          \
    hipLaunchKernelGGL(add_bias_kernel<T>, dim3(grid), dim3(256), 0, st, (T*)x, (const T*)bias, rows, cols); \
    MH_CHECK_LAUNCH();                                                                                        \
    return MH_OK;
    MH_DISPATCH_DTYPE(dtype, "mh_add_bias", MH_BIAS_CALL);
#undef MH_BIAS_CALL
}

}  // extern "C"
