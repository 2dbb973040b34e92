// Shared helpers for the gfx950 kernels: error plumbing, wave64 reductions,
// 16-bit float vector types.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>
#include <stdint.h>
#include <stddef.h>

#include "../../include/minit_hip.h"

namespace mh {

// Records a message for mh_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define MH_CHECK_HIP(expr)                                                        \
    do {                                                                          \
        hipError_t _e = (expr);                                                   \
        if (_e != hipSuccess)                                                     \
            return ::mh::fail(MH_ERR_HIP, "%s: %s", #expr, hipGetErrorString(_e)); \
    } while (0)

#define MH_REQUIRE(cond, ...)                                   \
    do {                                                        \
        if (!(cond)) return ::mh::fail(MH_ERR_INVALID, __VA_ARGS__); \
    } while (0)

// Launch-error check that does not synchronise.
#define MH_CHECK_LAUNCH() MH_CHECK_HIP(hipGetLastError())

inline hipStream_t as_stream(mh_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Number of compute units of the current device (cached per process).
int compute_units();
int f16_gemv_prepare();  // f16_matmul.hip: per-device set-up of the eight-row dot-product kernel

typedef _Float16 half_t;
// Buffer resource word 3 for raw (untyped, offset-addressed) buffer loads on gfx9:
// DATA_FORMAT = 32 bit; and the cache-policy operand of the buffer load builtins:
// bit 0 sc0, bit 1 nt, bit 4 sc1 (sc1 alone = agent scope).
constexpr int kBufferRsrcFlags = 0x00020000;
constexpr int kBufferStreamAgent = 2 | 16;

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef int int4_t __attribute__((ext_vector_type(4)));
typedef unsigned int uint4_t __attribute__((ext_vector_type(4)));
typedef unsigned int uint2_t __attribute__((ext_vector_type(2)));
typedef int int16_t_v __attribute__((ext_vector_type(16)));

constexpr int kWave = 64;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// Block-wide reductions over up to 16 waves; `smem` holds >= 16 floats and may
// be reused after the call returns (the helper syncs on both sides).
__device__ __forceinline__ float block_sum(float v, float* smem) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nwaves = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    float r = 0.f;
    for (int i = 0; i < nwaves; ++i) r += smem[i];
    return r;
}

__device__ __forceinline__ float block_max(float v, float* smem) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nwaves = (blockDim.x + 63) >> 6;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    float r = -INFINITY;
    for (int i = 0; i < nwaves; ++i) r = fmaxf(r, smem[i]);
    return r;
}

// ---- cross-workgroup hand-off without device-wide cache flushes ---------------------
// Split-K partial sums go from many workgroups to the one that finishes last.
// A release/acquire fence pair at agent scope would do, but on a multi-XCD part
// it writes back and invalidates a whole L2 per fence, once per workgroup.  The
// data are instead moved with agent-scope relaxed atomic stores and loads, which
// are written through to / fetched from the device-coherent level individually,
// and ordered by hand: every thread waits until its stores are acknowledged
// (s_waitcnt 0), the workgroup meets at a barrier, then one thread bumps the
// arrival counter with an agent-scope atomic.
__device__ __forceinline__ void store_agent(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_agent(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// 16-byte forms of the two above (the compiler has no vector atomics; sc1 is the
// agent-scope cache policy it gives the scalar ones).  The load is asynchronous:
// wait_agent_loads() must come between it and the first use of its result.
// (The two wait states behind the store: a vector instruction that overwrites the data registers of a
// store of more than 8 bytes within two wait states corrupts what some lanes store -- the compiler keeps
// that distance for its own stores and cannot see into this one.)
__device__ __forceinline__ void store_agent4(float* p, float4_t v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ float4_t load_agent4(const float* p) {
    float4_t v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
    return v;
}
template <int COUNT>
__device__ __forceinline__ void wait_agent_loads(float4_t (&v)[COUNT]) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < COUNT; ++i) asm volatile("" : "+v"(v[i]));  // uses of v[i] stay below the wait
}

// True, in every thread, for the workgroup that arrives last of `expected`; that
// workgroup also resets the counter for the next launch.  All threads of the
// workgroup must call it.
__device__ __forceinline__ bool arrive_and_check_last(unsigned* counter, unsigned expected, int* flag) {
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned prev = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int last = prev == expected - 1;
        if (last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag = last;
    }
    __syncthreads();
    return *flag != 0;
}

// Wave priority that falls as the wave's work gets done: `done` of `total` units behind it -> 3, 2, 1, 0
// by quarters (delay8: eighths of a unit of grace before the first step down).  Waves that share a SIMD --
// of one workgroup or of two on one CU -- are otherwise served oldest first, so the older one runs
// ahead and the younger one finishes alone; with this the one behind is served first.
// (s_setprio takes an immediate.)
__device__ __forceinline__ void set_priority_by_progress(int done, int total, int delay8 = 0) {
    const int level = 3 - min(3, max(done * 8 - delay8, 0) / (2 * total));
    if (level == 3) __builtin_amdgcn_s_setprio(3);
    else if (level == 2) __builtin_amdgcn_s_setprio(2);
    else if (level == 1) __builtin_amdgcn_s_setprio(1);
    else __builtin_amdgcn_s_setprio(0);
}

// 16-bit storage <-> fp32.
template <typename T> struct Cvt;
template <> struct Cvt<half_t> {
    static __device__ __forceinline__ float to_f32(half_t v) { return (float)v; }
    static __device__ __forceinline__ half_t from_f32(float v) { return (half_t)v; }
};
template <> struct Cvt<__hip_bfloat16> {
    static __device__ __forceinline__ float to_f32(__hip_bfloat16 v) { return __bfloat162float(v); }
    static __device__ __forceinline__ __hip_bfloat16 from_f32(float v) { return __float2bfloat16(v); }
};
template <> struct Cvt<float> {
    static __device__ __forceinline__ float to_f32(float v) { return v; }
    static __device__ __forceinline__ float from_f32(float v) { return v; }
};

}  // namespace mh
