// In-register GPTQ sub-word extraction and dequantisation.
//
// Arithmetic contract (minit/quantize/dispatch.py:14-20 of the reference, in
// fp16): W = (q - (z + 1)) * s.  q - (z + 1) is an exact small integer, so the
// multiply is the only rounding.  The extraction below builds that integer
// without int->float conversions: OR-ing a sub-word into the mantissa of the
// fp16 constant 1024 (0x6400) yields 1024 + q exactly (or 1024 + 16 q when the
// sub-word sits four bits up), and one packed subtract / fma against a
// per-column constant removes both the bias and the zero point.  Sub-word i of
// a word sits at bit i * bits (examples/qwen1_5_int8.py:107-116,129-136).
#pragma once

#include "common.h"

namespace mh {

#pragma clang fp contract(off)

__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
__device__ __forceinline__ uint32_t as_u32(half2_t h) { return __builtin_bit_cast(uint32_t, h); }

template <int BITS> struct Packing;
template <> struct Packing<4> {
    static constexpr int kPerWord = 8;
    static constexpr int kPairs = 4;
    static constexpr uint32_t kMask = 0xFu;
};
template <> struct Packing<8> {
    static constexpr int kPerWord = 4;
    static constexpr int kPairs = 2;
    static constexpr uint32_t kMask = 0xFFu;
};

// Per-(group, column) constants.
struct ColumnConst {
    half2_t scale;   // (s, s)
    half2_t zero_lo; // (1024 + z + 1) twice
    half2_t zero_hi; // (64 + z + 1) twice; 4-bit only
};

__device__ __forceinline__ ColumnConst make_column_const(half_t s, uint32_t z) {
    ColumnConst c;
    const half_t zp1 = (half_t)(float)(z + 1u);  // exact: z + 1 <= 256
    c.scale = half2_t{s, s};
    const half_t lo = (half_t)1024.0f + zp1;
    const half_t hi = (half_t)64.0f + zp1;
    c.zero_lo = half2_t{lo, lo};
    c.zero_hi = half2_t{hi, hi};
    return c;
}

// The same constants from the bits of s and the zero point, without conversions: below 2048 an fp16
// integer n + 1024 is the bit pattern 0x6400 + n, and 64 + n (n < 64) is 0x5400 + 16 n, so each pair is
// one multiply-add.  (8-bit zero points reach 256: zero_lo still holds, zero_hi is not used there.)
__device__ __forceinline__ ColumnConst column_const_from_bits(uint32_t sbits, uint32_t z) {
    ColumnConst c;
    c.scale = as_half2(sbits * 0x00010001u);
    c.zero_lo = as_half2((z + 1u) * 0x00010001u + 0x64006400u);
    c.zero_hi = as_half2((z + 1u) * 0x00100010u + 0x54005400u);
    return c;
}

// Bit masks and the fp16 bias kept in registers so that each extraction is a
// single v_and_or_b32 (VOP3 on gfx9 takes no literals; left as literals the
// compiler splits it into v_and + v_or).  Build once per kernel.
struct DequantRegs {
    uint32_t magic;    // 0x64006400: fp16 1024.0 twice
    uint32_t mask_lo;  // sub-word in mantissa bits 0..3 (or 0..7)
    uint32_t mask_hi;  // sub-word in mantissa bits 4..7; 4-bit only
    __device__ __forceinline__ void init(int bits) {
        magic = 0x64006400u;
        mask_lo = bits == 4 ? 0x000F000Fu : 0x00FF00FFu;
        mask_hi = 0x00F000F0u;
        asm volatile("" : "+v"(magic));
        asm volatile("" : "+s"(mask_lo));
        asm volatile("" : "+s"(mask_hi));
    }
};

// Dequantises one packed word of one column into kPairs half2 values.
// Element order ("pair order") for 4 bits: (k0,k4) (k1,k5) (k2,k6) (k3,k7);
// for 8 bits: (k0,k2) (k1,k3).  Callers pair the activations the same way.
template <int BITS>
__device__ __forceinline__ void dequant_word(uint32_t q, const ColumnConst& c, const DequantRegs& r,
                                             half2_t* w);

template <>
__device__ __forceinline__ void dequant_word<4>(uint32_t q, const ColumnConst& c, const DequantRegs& r,
                                                half2_t* w) {
    const half2_t sixteenth = half2_t{(half_t)0.0625f, (half_t)0.0625f};
    const uint32_t q8 = q >> 8;
    const half2_t p0 = as_half2((q & r.mask_lo) | r.magic);
    const half2_t p1 = as_half2((q & r.mask_hi) | r.magic);
    const half2_t p2 = as_half2((q8 & r.mask_lo) | r.magic);
    const half2_t p3 = as_half2((q8 & r.mask_hi) | r.magic);
    w[0] = (p0 - c.zero_lo) * c.scale;
    w[1] = __builtin_elementwise_fma(p1, sixteenth, -c.zero_hi) * c.scale;
    w[2] = (p2 - c.zero_lo) * c.scale;
    w[3] = __builtin_elementwise_fma(p3, sixteenth, -c.zero_hi) * c.scale;
}

template <>
__device__ __forceinline__ void dequant_word<8>(uint32_t q, const ColumnConst& c, const DequantRegs& r,
                                                half2_t* w) {
    const half2_t p0 = as_half2((q & r.mask_lo) | r.magic);
    const half2_t p1 = as_half2(((q >> 8) & r.mask_lo) | r.magic);
    w[0] = (p0 - c.zero_lo) * c.scale;
    w[1] = (p1 - c.zero_lo) * c.scale;
}

// Re-orders 2*kPairs consecutive activations (as packed 32-bit words holding
// two fp16 each) into the pair order of dequant_word.
template <int BITS>
__device__ __forceinline__ void pair_activations(const uint32_t* x, uint32_t* xp);

template <>
__device__ __forceinline__ void pair_activations<4>(const uint32_t* x, uint32_t* xp) {
    // x[0]=(k0,k1) x[1]=(k2,k3) x[2]=(k4,k5) x[3]=(k6,k7)
    xp[0] = (x[0] & 0xFFFFu) | (x[2] << 16);
    xp[1] = (x[0] >> 16) | (x[2] & 0xFFFF0000u);
    xp[2] = (x[1] & 0xFFFFu) | (x[3] << 16);
    xp[3] = (x[1] >> 16) | (x[3] & 0xFFFF0000u);
}

template <>
__device__ __forceinline__ void pair_activations<8>(const uint32_t* x, uint32_t* xp) {
    // x[0]=(k0,k1) x[1]=(k2,k3)
    xp[0] = (x[0] & 0xFFFFu) | (x[1] << 16);
    xp[1] = (x[0] >> 16) | (x[1] & 0xFFFF0000u);
}

// Epilogues of the quantized product.  kEpilogueSiluPairs: every 256-column
// tile holds 128 "gate" columns followed by the 128 matching "up" columns and
// the result has N / 2 columns, out[m, t*128 + c] = silu(y[m, t*256 + c]) *
// y[m, t*256 + 128 + c] with y rounded to fp16 first (what a separate
// SiLU*up pass over the fp16 product would read) and fp32 until the store.
// kEpilogueResidual: out is the residual stream itself, out[m, n] = fp16(out[m, n] +
// fp16(y[m, n])) (the fp16 add of the models, examples/llama3_70b.py:159-162), and
// the sum of squares of the new values over each 256-column tile is left in
// ssq_out[m, tile] for the consumer that normalises the row (SmallFuse).
constexpr int kEpilogueNone = 0;
constexpr int kEpilogueSiluPairs = 1;
constexpr int kEpilogueResidual = 2;
// kEpilogueRopeAppend: the product is the fused q|k|v projection of one new
// token per row, heads of 128 dims.  Query heads are rotated (interleaved pairs,
// minit/cuda/kernel/cuda/rope.py:58-73, at positions[m]) into q_out [M, QH, 128];
// key heads are rotated and value heads copied into the caches at that position
// (examples/llama3_70b.py:93-100): k_cache [M, KVH, T, 128], vt_cache
// [M, KVH, T / 64, 128, 64] (vt_offset).  Values are rounded to fp16 before the rotation, as when the
// projection is stored first.
constexpr int kEpilogueRopeAppend = 3;

// The V cache of the decode attention, per (row, KV head): tiles of 64 positions, [T / 64][D][64],
// T a multiple of 64.  The 64 positions x D dims a wave of the attention kernel reads per chunk
// are then D * 128 bytes in one piece, and a lane's eight consecutive positions of one dim stay 16
// bytes (dim-major over the whole cache, [D][T], the same chunk is D pieces of 128 bytes one cache
// length apart: 4.7 against 5.9 TB/s for that footprint, 50.7 -> 48.2 us per layer at 32 rows).
constexpr int kVTile = 64;
__device__ __forceinline__ size_t vt_offset(int d, int pos, int head_dim = 128) {
    return ((size_t)(pos / kVTile) * head_dim + d) * kVTile + pos % kVTile;
}

// Optional fusions of the small-M product kernel around RMSNorm
// (minit/cuda/kernel/cuda/rms_norm.py:69-89), which is split in two:
//   norm(h)[k] = (h[k] * w[k]) * (1 / sqrt(sum h^2 / K + eps)).
// A producer with kEpilogueResidual writes the new residual stream h, the
// element-wise half xw = fp16(h * next_norm_w) and per-piece sums of squares; a
// consumer given ssq_in takes xw as its activations and multiplies its fp32
// accumulators by the row factor at the end.  Against normalise-then-round the one
// fp16 rounding per activation moves from after both factors to after the first.
struct SmallFuse {
    const float* ssq_in = nullptr;   // [M, ssq_tiles]: consumer
    int ssq_tiles = 0;
    float eps = 0.f;
    float* ssq_out = nullptr;             // [M, pieces]: kEpilogueResidual
    const half_t* next_norm_w = nullptr;  // [N]
    half_t* xw_out = nullptr;             // [M, N]
    unsigned* xw_clamped = nullptr;       // optional: set to 1 when an element of xw left the fp16 range
    // y[m, n] = fp16(fp16(y[m, n]) + bias[n]), the two roundings of the reference's product followed by
    // `output += bias` (examples/qwen1_5_int8.py:311-317), before any epilogue (the activation of
    // kEpilogueSiluPairs, the rotation, the residual add) sees y
    const half_t* bias = nullptr;         // [N]
    // kEpilogueRopeAppend
    const float* rope_cos = nullptr;  // [T, 64]
    const float* rope_sin = nullptr;
    const int32_t* positions = nullptr;  // [M]
    half_t* q_out = nullptr;
    half_t* k_cache = nullptr;
    half_t* vt_cache = nullptr;
    int q_heads = 0, kv_heads = 0, max_seq = 0;
};

// xw = fp16(h * w) of the split norm, kept finite: where the reference's x / rms * w is of
// order w, h * w can leave the fp16 range for a very large residual channel (|h| above
// 65504 / w); the product then saturates at the largest finite value instead of becoming
// an infinity that would turn the whole row of the next product into NaN.  A saturated
// element makes that channel of the normalised row smaller in magnitude than the
// reference's (which stays exact): `clamped`, when given, is set to 1 so that the caller
// can tell such a step from an exact one.
template <typename V>
__device__ __forceinline__ V norm_weighted(V h, V w, unsigned* clamped) {
    const V hi = (half_t)65504.f - V{}, lo = -hi;
    const V p = h * w;
    const V c = __builtin_elementwise_max(__builtin_elementwise_min(p, hi), lo);
    if (clamped != nullptr) {
        bool any = false;
#pragma unroll
        for (unsigned e = 0; e < sizeof(V) / sizeof(half_t); ++e) any |= !(p[e] == c[e]);
        if (any) atomicOr(clamped, 1u);
    }
    return c;
}

__device__ __forceinline__ half_t silu_pair(half_t gate, half_t up) {
    const float g = (float)gate;
    return (half_t)(g / (1.f + expf(-g)) * (float)up);
}

// The workspace of the split-K kernels starts with one arrival counter per
// 256-column tile.  The caller zero-fills the workspace once; every launch
// leaves the counters at zero again.
// Sums of squares per piece -> the share of one lane of a 32-lane row group (pieces
// p0, p0 + 32, ...), added in that order.  The first 256 pieces are requested
// together (ssq_lane_load) -- a loop that loads and adds per iteration costs one
// memory round trip per 32 pieces, eight for the 256 pieces a hidden size of 8192
// leaves -- and may be requested ahead of other loads and summed after them.
struct SsqLane {
    float v[8];
};
__device__ __forceinline__ SsqLane ssq_lane_load(const float* __restrict__ row, int pieces, int p0) {
    SsqLane s;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int t = p0 + 32 * j;
        s.v[j] = t < pieces ? row[t] : 0.f;
    }
    return s;
}
__device__ __forceinline__ float ssq_lane_sum(const SsqLane& s, const float* __restrict__ row, int pieces, int p0) {
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) ss += s.v[j];
    for (int t = p0 + 256; t < pieces; t += 32) ss += row[t];
    return ss;
}

constexpr int kMaxTileCounters = 16384;
constexpr size_t kTileCounterBytes = kMaxTileCounters * sizeof(unsigned);

// Host-side argument validation shared by the GPTQ entry points.
int check_gptq_args(const char* who, const void* x, const void* qweight, const void* qzeros,
                    const void* scales, const void* out, int M, int N, int K, int group_size,
                    int bits);

}  // namespace mh
