/*
 * minit_hip.h -- C ABI of the MI355X (gfx950) quantized-linear hot path.
 *
 * Every entry point is `extern "C"`, takes plain pointers and sizes, never
 * throws and never allocates device memory behind the caller's back (the
 * mh_malloc family aside, which *is* the allocator).  Device pointers are
 * caller-owned.  `stream` is a hipStream_t passed as void*; NULL is the null
 * stream, which is what the reference's Python host passes to every kernel
 * (`kernel(None, ...)`, e.g. minit/cuda/dispatch.py:442).
 *
 * Return value: 0 on success, non-zero on failure; mh_last_error() then
 * returns a thread-local, NUL-terminated description.  The reference instead
 * throws std::runtime_error through its extern "C" launchers
 * (minit/cuda/allocator.py:21-27), which terminates the process.
 *
 * All matrices are dense row-major.  fp16 is IEEE binary16.
 */
#ifndef MINIT_HIP_H
#define MINIT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* mh_stream_t;
typedef void* mh_event_t;

#define MH_OK 0
#define MH_ERR_INVALID 1   /* bad argument / shape contract violated */
#define MH_ERR_HIP 2       /* a HIP runtime call failed              */
#define MH_ERR_WORKSPACE 3 /* workspace missing or too small         */

/* ---- library ------------------------------------------------------------ */

int mh_abi_version(void);
const char* mh_last_error(void);

/* ---- device runtime ------------------------------------------------------
 * Replaces the allocator shim minit/cuda/allocator.py:30-50
 * (allocate_cuda_memory / copy_cuda_memory / free_cuda_memory / sync_cuda /
 * reset), with an explicit stream and error codes.
 */
int mh_device_count(int* count);
int mh_device_info(int* compute_units, int* wavefront_size, size_t* total_mem,
                   size_t* lds_per_block, int* clock_khz, char* name, size_t name_len);
int mh_malloc(void** ptr, size_t bytes);
int mh_free(void* ptr);
int mh_host_malloc(void** ptr, size_t bytes); /* pinned host memory */
int mh_host_free(void* ptr);
int mh_memcpy(void* dst, const void* src, size_t bytes, mh_stream_t stream); /* any direction, async */
int mh_memset(void* dst, int value, size_t bytes, mh_stream_t stream);
int mh_stream_create(mh_stream_t* stream);
int mh_stream_destroy(mh_stream_t stream);
int mh_stream_synchronize(mh_stream_t stream);
int mh_device_synchronize(void);
int mh_event_create(mh_event_t* event);
int mh_event_destroy(mh_event_t event);
int mh_event_record(mh_event_t event, mh_stream_t stream);
int mh_event_synchronize(mh_event_t event);
int mh_event_elapsed_ms(float* ms, mh_event_t start, mh_event_t stop);
/* dst[i] = src[i], 16-byte vectors; the plain copy kernel the bandwidth
 * counters are calibrated against. bytes must be a multiple of 16. */
int mh_copy_kernel(mh_stream_t stream, const void* src, void* dst, size_t bytes);

/* ---- GPTQ sub-word unpack -------------------------------------------------
 * Replaces `unpack(x, axis)` (examples/qwen1_5_int8.py:40-50) and the
 * RowPackedMatrix / ColPackedMatrix accessors (:97-138), generic in `bits`
 * (4 or 8).  packed is int32 [rows, cols]; out is uint8
 * [rows * (32/bits), cols] for axis 0, [rows, cols * (32/bits)] for axis 1.
 */
/* out row j = qweight row perm[j] of the K unpacked rows, both packed along K ([K/P, N] int32):
 * the one-time repack of an act-order checkpoint whose rows are sorted by group
 * (examples/qwen1_5_int8.py:283-285 keeps g_idx and gathers per element at every product instead).
 * perm int32 [K] holds every row once (not checked; entries outside [0, K) are clamped); not in place. */
int mh_gptq_permute_rows(mh_stream_t stream, const int32_t* qweight, const int32_t* perm, int32_t* out, int N,
                         int K, int bits);
int mh_gptq_unpack(mh_stream_t stream, const int32_t* packed, uint8_t* out,
                   size_t rows, size_t cols, int axis, int bits);

/* ---- GPTQ dequantize --------------------------------------------------------
 * Replaces dispatch_dequantize (minit/quantize/dispatch.py:14-20) applied to
 * the packed checkpoint tensors: out[k, n] = fp16((q[k,n] - (z[g,n] + 1)) * s[g,n]),
 * g = g_idx[k] (g_idx == NULL means g = k / group_size; an entry outside
 * [0, K / group_size) is clamped into it).
 *   qweight int32 [K/P, N] (packed along K), qzeros int32 [G, N/P] (packed
 *   along N), scales fp16 [G, N], g_idx int32 [K] or NULL, out fp16 [K, N];
 *   P = 32 / bits, G = K / group_size.
 */
int mh_gptq_dequant(mh_stream_t stream, const int32_t* qweight, const int32_t* qzeros,
                    const void* scales, const int32_t* g_idx, void* out,
                    int N, int K, int group_size, int bits);

/* ---- GPTQ quantized linear ---------------------------------------------------
 * Replaces dispatch_quantized_matrix_multiply (minit/quantize/dispatch.py:8-11)
 * and the fused kernel qmm_* / quantized_matrix_multiply
 * (examples/qwen1_5_int8.py:202-203, :244-267):
 *   out[m, n] = fp16( sum_k fp32(x[m,k]) * fp32(W[k,n]) ),  W as in mh_gptq_dequant.
 * Shape contract (qwen1_5_int8.py:247-254): K == P * rows(qweight) == len(g_idx),
 * N == P * cols(qzeros) == cols(scales).  Additionally N % 8 == 0,
 * K % group_size == 0.
 *
 * workspace: device scratch of at least mh_gptq_workspace_bytes(M, N, K, ...)
 * bytes (arrival counters followed by fp32 split-K partial sums), 256-byte
 * aligned, zero-filled once by the caller after allocation: every call leaves
 * the counters at zero again, so the buffer is never cleared between calls.
 * May be NULL when the size query returns 0.  It may be shared by calls that
 * are ordered on one stream, never by concurrent calls.
 *
 * mh_gptq_gemv   wave64 VALU path, no MFMA; M <= MH_GPTQ_GEMV_MAX_M.
 * mh_gptq_gemm   fp16 MFMA path; any M >= 1; the packed weights of one matrix
 *                (K * N * bits / 8 bytes) must stay below 2 GiB, the kernels
 *                address them with 32-bit buffer offsets.
 * mh_gptq_matmul picks one of the two (or the act-order path when g_idx is a
 *                non-trivial permutation).
 */
#define MH_GPTQ_GEMV_MAX_M 4
size_t mh_gptq_workspace_bytes(int M, int N, int K, int group_size, int bits);
int mh_gptq_gemv(mh_stream_t stream, const void* x, const int32_t* qweight,
                 const int32_t* qzeros, const void* scales, const int32_t* g_idx,
                 void* out, int M, int N, int K, int group_size, int bits,
                 void* workspace, size_t workspace_bytes);
int mh_gptq_gemm(mh_stream_t stream, const void* x, const int32_t* qweight,
                 const int32_t* qzeros, const void* scales, const int32_t* g_idx,
                 void* out, int M, int N, int K, int group_size, int bits,
                 void* workspace, size_t workspace_bytes);
int mh_gptq_matmul(mh_stream_t stream, const void* x, const int32_t* qweight,
                   const int32_t* qzeros, const void* scales, const int32_t* g_idx,
                   void* out, int M, int N, int K, int group_size, int bits,
                   void* workspace, size_t workspace_bytes);

/* The product with the bias of QLinearWithBias.forward (examples/qwen1_5_int8.py:311-317:
 * `output = quantized_matrix_multiply(...)`, then `output += bias`, two launches and two fp16
 * roundings there): out[m, n] = fp16( fp16(y[m, n]) + bias[n] ), bias fp16 [N] or NULL (then
 * exactly mh_gptq_matmul).  The add rides on the product kernel's own stores -- one launch, or
 * two where K is split and a second stage adds the partial sums -- except for act-order
 * weights (g_idx) and group sizes other than 32 / 64 / 128 / 256, where it is a launch of its
 * own (mh_add_bias).  Workspace as for mh_gptq_matmul. */
int mh_gptq_linear(mh_stream_t stream, const void* x, const int32_t* qweight, const int32_t* qzeros,
                   const void* scales, const int32_t* g_idx, const void* bias, void* out,
                   int M, int N, int K, int group_size, int bits, void* workspace, size_t workspace_bytes);

/* mh_gptq_matmul for callers that cannot allocate device memory or pass a
 * workspace: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  The first call on a device looks up the address of the
 * built-in buffer (hipGetSymbolAddress), which a stream capture must not record:
 * make that call outside any capture (a call under capture before it fails with
 * MH_ERR_INVALID and records nothing); every later call may be captured.  No counterpart in the reference (its fused product
 * accumulates with atomics into a zeroed output and needs no scratch,
 * examples/qwen1_5_int8.py:198,263).  Same arguments and results as
 * mh_gptq_matmul without the workspace pair: the split-K counters and partial
 * sums live in a buffer of MH_GPTQ_STATIC_SCRATCH_BYTES that the library holds
 * in device memory on every GPU it runs on until the process ends.  The call
 * allocates and frees nothing.  A shape whose mh_gptq_workspace_bytes exceeds
 * that size is rejected with MH_ERR_WORKSPACE.  Every call on a GPU uses that
 * GPU's one buffer (of the device that is current at the call): calls that
 * overlap on one GPU -- different streams, or threads -- race on it and give
 * wrong sums; calls ordered on one stream are safe. */
#define MH_GPTQ_STATIC_SCRATCH_BYTES (24u << 20)
size_t mh_gptq_static_scratch_bytes(void);
int mh_gptq_matmul_static(mh_stream_t stream, const void* x, const int32_t* qweight,
                          const int32_t* qzeros, const void* scales, const int32_t* g_idx,
                          void* out, int M, int N, int K, int group_size, int bits);

/* The gate|up projection of a gated MLP with SiLU*up fused into the reduction of
 * the product (examples/llama3_70b.py:126-130 runs the product, sigmoid,
 * multiply, multiply as four launches).  The N = 2 * ffn columns are laid out
 * in blocks of 256: 128 gate columns followed by the 128 up columns of the same
 * positions (column t*256 + c is gate column t*128 + c, column t*256 + 128 + c
 * is up column t*128 + c; qzeros and scales permuted alike -- a load-time
 * permutation of whole 8-column words).  out is [M, N / 2]:
 *   out[m, t*128 + c] = fp16( silu(y[m, t*256 + c]) * y[m, t*256 + 128 + c] ),
 * y the fp16-rounded product, silu and the multiply in fp32.  N % 256 == 0.  It is
 * one launch up to 32 rows with group_size in {32, 64, 128, 256} (the epilogue runs
 * in the product's reduction) and, above 32 rows, for 4-bit weights with K a
 * multiple of 128 and at least 512 whose column tiles fill the GPU without a split
 * of K (the epilogue runs in the store of the 64-, 128- or 256-row blocks); otherwise the
 * product goes to the workspace and one more pass applies the epilogue.  The
 * workspace is always required:
 * mh_gptq_silu_pairs_workspace_bytes(M, N, K, ...) bytes, zero-filled once. */
size_t mh_gptq_silu_pairs_workspace_bytes(int M, int N, int K, int group_size, int bits);
int mh_gptq_matmul_silu_pairs(mh_stream_t stream, const void* x, const int32_t* qweight,
                              const int32_t* qzeros, const void* scales, void* out,
                              int M, int N, int K, int group_size, int bits,
                              void* workspace, size_t workspace_bytes);

/* ---- dense fp16 product --------------------------------------------------------
 * Replaces dispatch_matmul + minit_gemm (minit/cuda/dispatch.py:59-78,
 * minit/cuda/kernel/cublas.py:68-111) for batch == 1:
 *   out[m, n] = fp16( sum_k fp32(a[m,k]) * fp32(b[n,k]) ), b stored [N, K].
 */
int mh_f16_matmul_nk(mh_stream_t stream, const void* a, const void* b, void* out,
                     int M, int N, int K);
/* BatchMatrixMultiply (minit/cuda/dispatch.py:82-101: the whole batch in one strided library call,
 * e.g. the q.k^T and p.v products of a prefill, `einsum("bsnd,btnd->bnst")`): out[i] = a[i] @ b[i]^T
 * for i < batch with a [batch, M, K], b [batch, N, K], out [batch, M, N], all dense.  One launch
 * for the whole batch (at most 65535 matrices). */
int mh_f16_matmul_nk_batched(mh_stream_t stream, const void* a, const void* b, void* out,
                             int batch, int M, int N, int K);

/* ---- W8A8 int8 GEMM --------------------------------------------------------------
 * No counterpart in the reference (its "int8" model is weight-only,
 * examples/qwen1_5_int8.py:156-200); operand orientation follows the
 * reference's dense product, weight stored [N, K].
 *   acc[m, n] = sum_k int32(a[m,k]) * int32(w[n,k])                (exact)
 *   out[m, n] = fp16( fp32(acc[m,n]) * (a_scale[m] * w_scale[n]) )
 * acc_i32 may be NULL (accumulators are then not written out); out_f16 may be
 * NULL when only the accumulators are wanted.  K % 64 == 0.
 */
int mh_i8_gemm(mh_stream_t stream, const int8_t* a, const int8_t* w,
               const float* a_scale, const float* w_scale, void* out_f16,
               int32_t* acc_i32, int M, int N, int K);
/* out[n, k] = in[k, n]: one-time layout conversion for weights stored [K, N]. */
int mh_i8_transpose(mh_stream_t stream, const int8_t* in, int8_t* out, int rows, int cols);

/* ---- normalisation, rotary, softmax, reductions ---------------------------------------
 * Same view convention as the reference: the tensor is seen as [a, b, c] and
 * the operation runs along b.  dtype: 0 = fp16, 1 = bf16, 2 = fp32.
 */
#define MH_F16 0
#define MH_BF16 1
#define MH_F32 2

/* minit_rms_norm (minit/cuda/kernel/cuda/rms_norm.py:94):
 * out = T( x / sqrt(sum(x^2)/b + (float)eps) * w[b] ), fp32 internally. */
int mh_rms_norm(mh_stream_t stream, const void* in, const void* weight, void* out,
                size_t a, size_t b, size_t c, double eps, int dtype);

/* minit_rope (minit/cuda/kernel/cuda/rope.py:75): x is [bs, seq, nh, hs],
 * interleaved pairs rotated by fp32 tables.  positions == NULL: tables are
 * [seq, hs/2] indexed by the sequence index (the reference form).
 * positions != NULL: int32 [bs, seq]; tables are [nr_positions, hs/2] and row
 * positions[b, s] is used (must be < nr_positions). */
int mh_rope(mh_stream_t stream, const void* in, const float* freqs_cos,
            const float* freqs_sin, const int32_t* positions, void* out,
            size_t bs, size_t seq, size_t nh, size_t hs, int dtype);

/* minit_softmax (minit/cuda/kernel/cuda/softmax.py:109): softmax along b. */
int mh_softmax(mh_stream_t stream, const void* in, void* out,
               size_t a, size_t b, size_t c, int dtype);

/* Softmax with the models' causal mask and 1/sqrt(d) scale fused in
 * (examples/llama3_70b.py:102-112): in is [rows_outer, s, t] with
 * t == offset + s; out[., i, j] = softmax_j( T(in * scale) + m[i, j] ),
 * m[i, j] = -inf iff j - offset > i.  scale == 1 skips the multiply. */
int mh_softmax_causal(mh_stream_t stream, const void* in, void* out,
                      size_t rows_outer, size_t s, size_t t, size_t offset,
                      float scale, int dtype);

/* minit_sum / minit_max (minit/cuda/kernel/cuda/reduce.py:95): [a,b,c] -> [a,1,c]. */
int mh_sum(mh_stream_t stream, const void* in, void* out, size_t a, size_t b, size_t c, int dtype);
int mh_max(mh_stream_t stream, const void* in, void* out, size_t a, size_t b, size_t c, int dtype);
/* mean along b as the reference composes it (minit/functional/reduce.py:14-18:
 * sum, then divide by a tensor filled with the axis length, both in T):
 * out = T( T(sum) / T(b) ), b > 0. */
int mh_mean(mh_stream_t stream, const void* in, void* out, size_t a, size_t b, size_t c, int dtype);

/* The element-wise kernels the models' silu is made of (examples/llama3_70b.py:44-45,
 * `x * F.sigmoid(x)`): the reference's Sigmoid expression, 1.0 / (1.0 + expf((float)-x))
 * evaluated in double and rounded once to T (minit/cuda/dispatch.py:143), and the
 * element-wise product in T (`{0} * {1}`, :137).  n elements, same shape. */
int mh_sigmoid(mh_stream_t stream, const void* in, void* out, size_t n, int dtype);
int mh_multiply(mh_stream_t stream, const void* a, const void* b, void* out, size_t n, int dtype);
/* The residual add of the models (`x = x + attn(...)`, examples/llama3_70b.py:159-162;
 * `{0} + {1}` in T, minit/cuda/dispatch.py:135): out = T(a + b), same shape. */
int mh_add(mh_stream_t stream, const void* a, const void* b, void* out, size_t n, int dtype);

/* silu(gate) * up in one pass (the models run sigmoid, multiply, multiply as
 * three launches: examples/llama3_70b.py:44-45,126-130,
 * minit/cuda/dispatch.py:137,143).  exact != 0 reproduces the three fp16
 * roundings of that sequence; exact == 0 keeps fp32 until the store. */
int mh_silu_mul(mh_stream_t stream, const void* gate, const void* up, void* out,
                size_t n, int exact, int dtype);

/* The bias of a quantized linear (QLinearWithBias.forward,
 * examples/qwen1_5_int8.py:311-317: the product, then `output += bias` with the
 * bias broadcast over the leading axes): x[r, c] = T(x[r, c] + bias[c]) in
 * place, one rounding in the storage type like the reference's Add kernel. */
int mh_add_bias(mh_stream_t stream, void* x, const void* bias, size_t rows, size_t cols, int dtype);

/* Activations in the row order of an act-order weight that was sorted by group
 * once at load time (the reference gathers scale and zero point per element of K
 * through g_idx instead, minit/quantize/dispatch.py:16-19; with W_sorted[j] =
 * W[index[j]] the product x W equals gather(x) W_sorted and W_sorted has
 * sequential groups): out[r, j] = x[r, index[j]], index int32 [cols], not in place. */
int mh_gather_columns(mh_stream_t stream, const void* x, const int32_t* index, void* out, size_t rows, size_t cols,
                      int dtype);

/* ---- Llama-family GPTQ decode loop ------------------------------------------------------
 * The callers around the quantized linears: one greedy decode step per token as
 * the reference's models run it (examples/llama3_70b.py:77-162,215-249;
 * sampling minit/chat/sample.py:11-14), enqueued from native code.  All
 * pointers are device pointers owned by the caller.
 *   qkv      fused q|k|v projection, GPTQ, [hidden] -> [(QH + 2 KVH) * D]
 *   gate_up  fused gate|up projection, [hidden] -> [2 * ffn], columns interleaved in
 *            blocks of 128 gate / 128 up as for mh_gptq_matmul_silu_pairs (ffn % 128 == 0);
 *            the activation is silu(gate) * up (for examples/qwen1_5_int8.py:376-385 gate is w2
 *            and up is w1)
 *   k_cache  fp16 [batch_max, KVH, max_seq, D], v_cache fp16 [batch_max, KVH, max_seq / 64, D, 64]
 *            (V is kept with positions contiguous, in tiles of 64, for the P.V matrix product:
 *            value d of position p sits at ((p / 64) * D + d) * 64 + p % 64 of its row and KV
 *            head); both appended in place; max_seq is a multiple of 64
 *   embed, lm_head     fp16 [vocab, hidden]; norms fp16 [hidden]
 *   freqs_cos / sin    fp32 [max_seq, D / 2]
 */
/* The attention core of one decode step on its own (examples/llama3_70b.py:77-113
 * for one new token per row: cache append, q.k^T, / sqrt(d), the causal mask --
 * identically zero here --, softmax, P.V), grouped-query heads sharing one read of
 * their KV head's cache instead of the reference's 8x head-expanded copies.
 *   mh_rope_kv_append   qkv fp16 [batch, (QH + 2 KVH) * D] (q heads, then k heads, then
 *                       v heads): q and k rotated at positions[b] with the interleaved
 *                       pairs of mh_rope, q to q_out [batch, QH, D], k into k_cache
 *                       [batch, KVH, max_seq, D] and v into vt_cache [batch, KVH,
 *                       max_seq / 64, D, 64] (the tiled layout of v_cache above) at that
 *                       position (clamped to the cache); max_seq a multiple of 64
 *   mh_attn_decode      out[b, h] = softmax(q[b, h] . K[b, h / (QH / KVH), 0..positions[b]] / sqrt(D)) . V,
 *                       fp32 inside, one rounding; D == 128, QH / KVH in {1, 2, 4, 8};
 *                       positions[b] is the index of the newest cache entry; cache
 *                       entries past it are never part of the result, whatever they hold.
 *                       The workspace is zero-filled once by the caller and left with its
 *                       counters at zero; where the counters end depends on batch and
 *                       KVH, so a workspace that moves to a call with other sizes is
 *                       zero-filled again. */
/* The residual add and the norm that follows it in one pass over the row
 * (examples/llama3_70b.py:159-162: `x = x + attn(...)`, then `norm(x)`): h[r, :] =
 * fp16(h + delta) in place (skipped when delta is NULL), out[r, :] = RMSNorm(h) *
 * weight with mh_rms_norm's arithmetic.  fp16, hidden a multiple of 8 up to 8192. */
int mh_add_rms_norm(mh_stream_t stream, void* h, const void* delta, const void* weight, void* out, int rows,
                    int hidden, float eps);
/* Greedy sampling on the device: out[r] = index of the first maximum of the fp16
 * row logits[r, 0..cols) (Top1Sampler, minit/chat/sample.py:11-14, which copies the
 * row to the host for numpy's argmax); NaN entries are never selected. */
int mh_argmax(mh_stream_t stream, const void* logits, int32_t* out, int rows, int cols);
size_t mh_attn_decode_workspace_bytes(int batch, int n_q_heads, int n_kv_heads, int head_dim, int max_seq);
int mh_attn_decode(mh_stream_t stream, const void* q, const void* k_cache, const void* vt_cache,
                   const int32_t* positions, void* out, int batch, int n_q_heads, int n_kv_heads, int head_dim,
                   int max_seq, void* workspace, size_t workspace_bytes);
int mh_rope_kv_append(mh_stream_t stream, const void* qkv, const float* freqs_cos, const float* freqs_sin,
                      const int32_t* positions, void* q_out, void* k_cache, void* vt_cache, int batch, int n_q_heads,
                      int n_kv_heads, int head_dim, int max_seq);

typedef struct {
    int n_layers, hidden, n_q_heads, n_kv_heads, head_dim, ffn, vocab;
    int group_size, bits, max_seq;
    float rms_eps;
} mh_llama_config;
/* One quantized linear of the model.  bias: fp16 [N] or NULL, added to the fp16-rounded product before
 * anything else sees it (QLinearWithBias.forward, examples/qwen1_5_int8.py:311-317; every linear of that
 * file's model has one); for gate_up it is interleaved like the columns.  perm: NULL for sequential
 * groups; for an act-order checkpoint (g_idx a permutation, :283-285) the caller sorts the rows of
 * qweight by group once at load time (mh_gptq_permute_rows) and passes the row order here, int32 [K]
 * with row j of qweight = row perm[j] of the checkpoint's: the loop then gathers the activations into
 * that order (mh_gather_columns) in front of the product. */
typedef struct {
    const int32_t* qweight;
    const int32_t* qzeros;
    const void* scales;
    const void* bias;
    const int32_t* perm;
} mh_qlinear;
typedef struct {
    mh_qlinear qkv, o, gate_up, down;
    const void* input_norm;
    const void* post_norm;
    void* k_cache;
    void* v_cache;
} mh_llama_layer;
int mh_llama_create(void** handle, const mh_llama_config* cfg);
int mh_llama_destroy(void* handle);
int mh_llama_set_layer(void* handle, int layer, const mh_llama_layer* l);
int mh_llama_set_globals(void* handle, const void* embed, const void* lm_head, const void* final_norm,
                         const float* freqs_cos, const float* freqs_sin);
/* Scratch for activations, split-K partials and counters; zero-fill it once. */
size_t mh_llama_scratch_bytes(void* handle, int batch);
/* Whether a fused residual + RMSNorm launch of the loop has saturated since `scratch` was zero-filled:
 * those launches keep fp16(h * norm_weight) and apply the row's 1 / rms in the consuming product
 * (the reference rounds x / rms * w once, rms_norm.py:69-89), and a residual channel with
 * |h * w| > 65504 is held at the largest finite fp16 value there, which makes that channel of the
 * normalised row smaller than the reference's.  *clamped is 1 after such a step (the decoded tokens
 * then carry no parity claim), 0 otherwise; waits for `stream`.  Same batch and scratch as the decode
 * calls. */
int mh_llama_norm_clamped(void* handle, mh_stream_t stream, int batch, const void* scratch, int32_t* clamped);
/* Runs n_steps greedy steps.  tokens [batch] int32 holds the input token of the
 * first step and the last sampled token on return; positions [batch] int32 is
 * where each row's next K/V entry goes and is advanced by one per step;
 * out_tokens (optional) receives [n_steps, batch]; logits_out (optional)
 * receives the last step's fp16 logits [batch, vocab].  The caller keeps
 * positions[b] + n_steps <= max_seq; the kernels clamp a position to
 * [0, max_seq - 1], so a cache that is full overwrites its last slot (wrong
 * tokens, no access outside the cache). */
int mh_llama_decode(void* handle, mh_stream_t stream, int batch, int32_t* tokens, int32_t* positions,
                    int n_steps, int32_t* out_tokens, void* logits_out, void* scratch, size_t scratch_bytes);
/* The same, with one step recorded into a HIP graph on first use and replayed
 * n_steps times (the reference's hook for replaying a recorded operator sequence
 * is minit/trace/executor.py:49-119, which still dispatches and allocates per
 * operator; here a step has no host work at all).  Same arguments and results;
 * `stream` must be a created stream (the null stream cannot record).  The
 * recorded step is kept in the handle, keyed by (batch, tokens, positions,
 * out_tokens, scratch), until the model's pointers are set again or it is
 * destroyed; those buffers must stay allocated while it is kept. */
int mh_llama_decode_graph(void* handle, mh_stream_t stream, int batch, int32_t* tokens, int32_t* positions,
                          int n_steps, int32_t* out_tokens, void* logits_out, void* scratch, size_t scratch_bytes);

/* ---- synthetic inputs ------------------------------------------------------------------
 * No counterpart in the reference (it loads checkpoints from disk,
 * minit/module/checkpoint.py:11-44).  Counter-based generators that fill device
 * buffers for benchmarks: uniform 32-bit words (= uniform 4-bit weights),
 * sub-words uniform in [lo, hi] (zero points), N(mean, std) optionally folded
 * and offset (scales, activations), uniform int8.
 */
int mh_synth_u32(mh_stream_t stream, uint32_t* out, size_t n, uint64_t seed);
int mh_synth_subwords(mh_stream_t stream, uint32_t* out, size_t n, int bits, uint32_t lo, uint32_t hi,
                      uint64_t seed);
int mh_synth_normal(mh_stream_t stream, void* out, size_t n, float mean, float std, int take_abs,
                    float offset, uint64_t seed, int dtype);
int mh_synth_i8(mh_stream_t stream, int8_t* out, size_t n, int lo, int hi, uint64_t seed);

#ifdef __cplusplus
}
#endif
#endif /* MINIT_HIP_H */
