// Instruction-issue calibration for the GPTQ MFMA kernels (no counterpart in the
// reference): a register-resident loop that issues, per iteration and wave, NV packed
// fp16 vector instructions (the kind the in-register dequantisation is made of) and NM
// v_mfma_f32_16x16x32_f16, with no memory traffic.  Timed with one, two and four waves
// per SIMD it answers whether vector and matrix instructions of the waves of one SIMD
// overlap or queue behind each other, which sets the issue-bound ceiling of a kernel
// that needs 13 vector instructions per packed word next to one MFMA per 64 words.
#include "common.h"

namespace mh {

// DEP: the MFMA's B operand is built from the vector results of the same iteration (as
// in the real kernel, where the dequantised words feed the MFMA); otherwise constant.
template <int NV, int NM, bool DEP>
__global__ void __launch_bounds__(256) issue_probe_kernel(float* __restrict__ out, int iters, half2_t a) {
    half2_t x[12];
#pragma unroll
    for (int i = 0; i < 12; ++i) x[i] = half2_t{(half_t)(float)(threadIdx.x & 7), (half_t)(float)i};
    float4_t acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    half8_t av;
#pragma unroll
    for (int i = 0; i < 8; ++i) av[i] = (half_t)(0.01f * i);
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < NV; ++i) x[i % 12] = x[i % 12] * a;     // v_pk_mul_f16 on 12 independent chains
#pragma unroll
        for (int i = 0; i < NM; ++i) {
            half8_t b = av;
            if (DEP) {
                const half2_t p0 = x[(i * 3) % 12], p1 = x[(i * 3 + 1) % 12], p2 = x[(i * 3 + 2) % 12];
                b = half8_t{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p0[0], p0[1]};
            }
            acc[i % 4] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, b, acc[i % 4], 0, 0, 0);
        }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 12; ++i) s += (float)x[i][0] + (float)x[i][1];
#pragma unroll
    for (int i = 0; i < 4; ++i) s += acc[i][0] + acc[i][3];
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// Cost of a device-wide barrier between the phases of a would-be persistent kernel, against the cost
// of a kernel boundary: every workgroup bumps one agent-scope counter and polls it until all have
// arrived, `rounds` times.  The counter only grows (round r waits for (r + 1) * workgroups), so no
// reset races with a late reader.  Every wait is bounded: after spin_limit polls a workgroup sets
// the error word and, like every workgroup that sees it set, stops waiting for the rest of the
// launch, so all waves exit whether or not the workgroups were resident together.
// groups > 1: two levels.  Workgroup b arrives at counter[32 * (1 + b % groups)] (a line of its own per
// group; consecutive workgroups go to different XCDs, so a group is the workgroups of one XCD when
// groups is 8), and the one that completes its group's round bumps counter[0], which everybody polls:
// the arrivals at one address, which serialise, drop from all workgroups to the group size plus groups.
__global__ void __launch_bounds__(256) grid_barrier_probe_kernel(unsigned* __restrict__ counter,
                                                                 unsigned* __restrict__ error, int rounds,
                                                                 int spin_limit, int groups) {
    __shared__ int give_up;
    if (threadIdx.x == 0) give_up = 0;
    __syncthreads();
    const unsigned group = blockIdx.x % groups;
    const unsigned group_size = gridDim.x / groups + (group < gridDim.x % groups ? 1u : 0u);
    for (int r = 0; r < rounds; ++r) {
        if (threadIdx.x == 0 && !give_up) {
            if (groups > 1) {
                const unsigned prev = __hip_atomic_fetch_add(counter + 32 * (1 + group), 1u, __ATOMIC_RELAXED,
                                                             __HIP_MEMORY_SCOPE_AGENT);
                if (prev + 1 == (unsigned)(r + 1) * group_size)
                    __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else {
                __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            const unsigned target = (unsigned)(r + 1) * (groups > 1 ? (unsigned)groups : gridDim.x);
            int spins = 0;
            while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
                if (++spins > spin_limit || __hip_atomic_load(error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) {
                    __hip_atomic_store(error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    give_up = 1;
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
        }
        __syncthreads();
    }
}

// Read-only copy of the small-M kernel's weight stream: workgroup (tile, part) of four waves walks
// rows_per_block packed rows of a 256-column tile; a wave load is four packed rows x 256 bytes (lane / 16 =
// row, lane % 16 = four adjacent columns), eight loads in flight per wave, streaming hint.  What this reaches
// is what the memory system delivers to that footprint with no arithmetic in the way.
__global__ void __launch_bounds__(256) weight_stream_probe_kernel(const uint32_t* __restrict__ w,
                                                                  uint32_t* __restrict__ sink, int N,
                                                                  int rows_per_block) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t* p = w + (size_t)blockIdx.y * rows_per_block * N + blockIdx.x * 256 + (size_t)(lane >> 4) * N +
                        wave * 64 + (lane & 15) * 4;
    const int steps = rows_per_block / 4;
    uint4_t acc = {0u, 0u, 0u, 0u}, ring[8];
#pragma unroll
    for (int d = 0; d < 8; ++d)
        ring[d] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(p + (size_t)min(d, steps - 1) * 4 * N));
    for (int s = 0; s < steps; s += 8) {
#pragma unroll
        for (int d = 0; d < 8; ++d) {
            acc ^= ring[d];
            ring[d] = __builtin_nontemporal_load(
                reinterpret_cast<const uint4_t*>(p + (size_t)min(s + d + 8, steps - 1) * 4 * N));  // the tail re-reads the last rows
        }
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) sink[threadIdx.x] = 1u;  // keeps the loads alive
}

__global__ void __launch_bounds__(256) empty_probe_kernel(unsigned* __restrict__ sink) {
    if (sink == nullptr) return;
    if (threadIdx.x == 0 && blockIdx.x == 0x7fffffffu) *sink = 1u;  // never true: keeps the argument alive
}

}  // namespace mh

using namespace mh;

extern "C" int mh_grid_barrier_probe(mh_stream_t stream, unsigned* counter, unsigned* error, int blocks, int rounds,
                                     int spin_limit, int groups) {
    MH_REQUIRE(counter != nullptr && error != nullptr && blocks > 0 && rounds > 0 && spin_limit > 0 && groups >= 1 &&
                   groups <= 16 && groups <= blocks,
               "mh_grid_barrier_probe: bad argument");
    MH_REQUIRE(blocks <= compute_units() * 2, "mh_grid_barrier_probe: %d workgroups cannot be resident together on %d CUs",
               blocks, compute_units());
    MH_REQUIRE((long)blocks * rounds < (1L << 31), "mh_grid_barrier_probe: counter would overflow");
    grid_barrier_probe_kernel<<<blocks, 256, 0, as_stream(stream)>>>(counter, error, rounds, spin_limit, groups);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

extern "C" int mh_weight_stream_probe(mh_stream_t stream, const uint32_t* words, uint32_t* sink, int rows, int N,
                                      int parts) {
    MH_REQUIRE(words != nullptr && sink != nullptr && rows > 0 && N > 0 && parts > 0, "mh_weight_stream_probe: bad argument");
    MH_REQUIRE(N % 256 == 0 && rows % (parts * 32) == 0, "mh_weight_stream_probe: N %% 256 == 0 and rows %% (32 * parts) == 0");
    weight_stream_probe_kernel<<<dim3(N / 256, parts), 256, 0, as_stream(stream)>>>(words, sink, N, rows / parts);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

extern "C" int mh_empty_probe(mh_stream_t stream, unsigned* sink, int blocks) {
    MH_REQUIRE(blocks > 0, "mh_empty_probe: bad argument");
    empty_probe_kernel<<<blocks, 256, 0, as_stream(stream)>>>(sink);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

extern "C" int mh_issue_probe(mh_stream_t stream, float* out, int blocks, int iters, int n_valu, int n_mfma,
                              int dependent) {
    MH_REQUIRE(out != nullptr && blocks > 0 && iters > 0, "mh_issue_probe: bad argument");
    const half2_t a = half2_t{(half_t)1.001f, (half_t)0.999f};
    hipStream_t s = as_stream(stream);
#define MH_PROBE(NV, NM, DEP)                                                         \
    if (n_valu == NV && n_mfma == NM && (dependent != 0) == DEP) {                     \
        issue_probe_kernel<NV, NM, DEP><<<blocks, 256, 0, s>>>(out, iters, a);         \
        MH_CHECK_LAUNCH();                                                             \
        return MH_OK;                                                                  \
    }
    MH_PROBE(52, 0, false)
    MH_PROBE(0, 4, false)
    MH_PROBE(52, 4, false)
    MH_PROBE(52, 4, true)
    MH_PROBE(26, 4, true)
    MH_PROBE(104, 4, true)
    MH_PROBE(0, 8, false)
#undef MH_PROBE
    return fail(MH_ERR_INVALID, "mh_issue_probe: no instance for %d vector + %d matrix instructions (dependent=%d)",
                n_valu, n_mfma, dependent);
}
