// Device-side generation of synthetic benchmark inputs (counter-based hashing,
// so any element can be regenerated from its index and the seed).  Filling
// 35 GB of 70B-shape weights from the host would take minutes; these kernels
// write them at HBM speed.  Not part of the quantized-linear arithmetic.
#include "common.h"

namespace mh {

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__device__ __forceinline__ float uniform01(uint32_t bits) {  // (0, 1]
    return ((float)(bits >> 8) + 1.0f) * (1.0f / 16777216.0f);
}

__global__ void synth_u32_kernel(uint32_t* out, size_t n, uint64_t seed) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        out[i] = (uint32_t)(mix64(seed * 0x100000001B3ull + i) >> 16);
}

// every `bits`-wide sub-word of every output word uniform in [lo, hi]
__global__ void synth_subwords_kernel(uint32_t* out, size_t n, int bits, uint32_t lo, uint32_t hi,
                                      uint64_t seed) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const int per_word = 32 / bits;
    const uint32_t span = hi - lo + 1;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        uint32_t word = 0;
        for (int j = 0; j < per_word; ++j) {
            const uint64_t h = mix64(seed * 0x100000001B3ull + i * per_word + j);
            word |= (lo + (uint32_t)((h >> 20) % span)) << (j * bits);
        }
        out[i] = word;
    }
}

// out = fp16( offset + (take_abs ? |N(mean, std)| : N(mean, std)) )
__global__ void synth_normal_f16_kernel(half_t* out, size_t n, float mean, float std, int take_abs,
                                        float offset, uint64_t seed) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const uint64_t h = mix64(seed * 0x100000001B3ull + i);
        const float u1 = uniform01((uint32_t)h), u2 = uniform01((uint32_t)(h >> 32));
        float z = mean + std * sqrtf(-2.0f * logf(u1)) * cosf(6.2831853071795865f * u2);
        if (take_abs) z = fabsf(z);
        out[i] = (half_t)(z + offset);
    }
}

__global__ void synth_normal_f32_kernel(float* out, size_t n, float mean, float std, int take_abs,
                                        float offset, uint64_t seed) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const uint64_t h = mix64(seed * 0x100000001B3ull + i);
        const float u1 = uniform01((uint32_t)h), u2 = uniform01((uint32_t)(h >> 32));
        float z = mean + std * sqrtf(-2.0f * logf(u1)) * cosf(6.2831853071795865f * u2);
        if (take_abs) z = fabsf(z);
        out[i] = z + offset;
    }
}

__global__ void synth_i8_kernel(int8_t* out, size_t n, int lo, int hi, uint64_t seed) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const uint32_t span = (uint32_t)(hi - lo + 1);
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        out[i] = (int8_t)(lo + (int)((mix64(seed * 0x100000001B3ull + i) >> 20) % span));
}

static unsigned synth_grid(size_t n) {
    size_t blocks = (n + 255) / 256;
    const size_t cap = (size_t)compute_units() * 32;
    if (blocks > cap) blocks = cap;
    return (unsigned)(blocks ? blocks : 1);
}

}  // namespace mh

using namespace mh;

extern "C" {

int mh_synth_u32(mh_stream_t stream, uint32_t* out, size_t n, uint64_t seed) {
    if (n == 0) return MH_OK;
    MH_REQUIRE(out != nullptr, "mh_synth_u32: null pointer");
    hipLaunchKernelGGL(synth_u32_kernel, dim3(synth_grid(n)), dim3(256), 0, as_stream(stream), out, n, seed);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

int mh_synth_subwords(mh_stream_t stream, uint32_t* out, size_t n, int bits, uint32_t lo, uint32_t hi,
                      uint64_t seed) {
    if (n == 0) return MH_OK;
    MH_REQUIRE(out != nullptr, "mh_synth_subwords: null pointer");
    MH_REQUIRE(bits == 4 || bits == 8, "mh_synth_subwords: bits must be 4 or 8");
    MH_REQUIRE(lo <= hi && hi < (1u << bits), "mh_synth_subwords: bad range [%u, %u]", lo, hi);
    hipLaunchKernelGGL(synth_subwords_kernel, dim3(synth_grid(n)), dim3(256), 0, as_stream(stream), out, n,
                       bits, lo, hi, seed);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

int mh_synth_normal(mh_stream_t stream, void* out, size_t n, float mean, float std, int take_abs,
                    float offset, uint64_t seed, int dtype) {
    if (n == 0) return MH_OK;
    MH_REQUIRE(out != nullptr, "mh_synth_normal: null pointer");
    MH_REQUIRE(dtype == MH_F16 || dtype == MH_F32, "mh_synth_normal: dtype must be fp16 or fp32");
    if (dtype == MH_F16)
        hipLaunchKernelGGL(synth_normal_f16_kernel, dim3(synth_grid(n)), dim3(256), 0, as_stream(stream),
                           (half_t*)out, n, mean, std, take_abs, offset, seed);
    else
        hipLaunchKernelGGL(synth_normal_f32_kernel, dim3(synth_grid(n)), dim3(256), 0, as_stream(stream),
                           (float*)out, n, mean, std, take_abs, offset, seed);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

int mh_synth_i8(mh_stream_t stream, int8_t* out, size_t n, int lo, int hi, uint64_t seed) {
    if (n == 0) return MH_OK;
    MH_REQUIRE(out != nullptr, "mh_synth_i8: null pointer");
    MH_REQUIRE(lo <= hi && lo >= -128 && hi <= 127, "mh_synth_i8: bad range");
    hipLaunchKernelGGL(synth_i8_kernel, dim3(synth_grid(n)), dim3(256), 0, as_stream(stream), out, n, lo, hi,
                       seed);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

}  // extern "C"
