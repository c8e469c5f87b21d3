/*
 * tpamd.h - C ABI of the MI355X (gfx950) hot path of a tensor-parallel transformer layer:
 * state-dict slicing, rank-shard Linears and the single-device partial-sum reduction.
 *
 * The reference implementation (BlackSamorez/tensor_parallel) is pure Python and has no FFI.
 * Each entry point below names the Python call of the reference whose work it performs.
 *
 * Conventions
 *   - every pointer named *_dev is device memory of the current HIP device; everything else is host memory;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); all work is enqueued on it
 *     and the call returns without waiting for it;
 *   - matrices are row-major with an explicit leading dimension in ELEMENTS;
 *   - return value: 0 on success, a negative tpamd_status otherwise; tpamd_last_error() then returns a
 *     message for the calling thread;
 *   - every entry point may be called concurrently from several host threads. Besides the thread-local error
 *     message the library keeps one piece of state: tpamd_linear / tpamd_linear_add / tpamd_swiglu_up split K for
 *     shapes with few output tiles (M from 17 to a few thousand, decided by a cost model), tpamd_linear_w8 does so
 *     from 2 rows on large matrices, tpamd_attention splits long key ranges, and they keep fp32 scratch buffers for
 *     the partial results: one per (device, stream), 64 MiB on a 256-CU part, allocated with hipMalloc at the
 *     stream's first such call and kept until the process ends (at most 32 streams per device get one; calls on
 *     further streams run unsplit). Streams never share a buffer, so such calls on different streams of a device
 *     need no ordering among themselves. Nothing can be allocated while a stream is being captured: the first
 *     allocation on a device therefore sets one spare buffer aside, which the first capturing stream without a
 *     buffer of its own takes over; a capture that finds neither runs the call unsplit (slower, same result up to
 *     summation order). A captured graph keeps using the buffer of the stream it was captured on: replaying it
 *     on another stream while the capture stream runs K-split work is for the caller to order.
 *   - tuning knobs (environment variables TPAMD_*) are read once, when the library is loaded.
 */
#ifndef TPAMD_H
#define TPAMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TPAMD_ABI_VERSION 5

typedef enum tpamd_status {
    TPAMD_OK = 0,
    TPAMD_ERR_INVALID = -1,     /* bad argument (shape, alignment, dtype, null pointer) */
    TPAMD_ERR_UNSUPPORTED = -2, /* legal request this build has no kernel for */
    TPAMD_ERR_HIP = -3,         /* a HIP runtime call failed */
    TPAMD_ERR_NOMEM = -4        /* host or device allocation failed */
} tpamd_status;

typedef enum tpamd_dtype {
    TPAMD_BF16 = 0,
    TPAMD_F16 = 1,
    TPAMD_F32 = 2
} tpamd_dtype;

/* How tpamd_reduce_partials accumulates. */
typedef enum tpamd_accum {
    /* ((p0 + p1) + p2) + ... with the running sum rounded to the tensor dtype after every add:
     * the arithmetic of the reference's CPU reduction, `sum([...])` over same-dtype tensors
     * (src/tensor_parallel/cross_device_ops.py:49), taken in rank order. */
    TPAMD_ACCUM_STEPWISE = 0,
    /* fp32 running sum over ranks 0..W-1, one rounding at the store. */
    TPAMD_ACCUM_F32 = 1
} tpamd_accum;

/* Epilogue applied by the shard Linears before the store. */
typedef enum tpamd_act {
    TPAMD_ACT_NONE = 0,
    TPAMD_ACT_GELU = 1 /* exact erf GELU */
} tpamd_act;

int tpamd_abi_version(void);
const char *tpamd_last_error(void);
/* Reads the TPAMD_* environment variables again (they are read once at load time otherwise). For tests and
 * experiments that force a kernel variant; no counterpart in the reference. Not synchronised: call it while no other
 * thread is inside the library. */
void tpamd_tuning_reload(void);
/* The K-split scratch buffer that work on `stream` of the current device uses: *ptr_out = NULL and *bytes_out = 0
 * while the stream has none. Diagnostic; no counterpart in the reference. */
int tpamd_scratch_query(void *stream, void **ptr_out, uint64_t *bytes_out);
/* Gives back the scratch buffer of `stream` on the current device (no-op when it has none): call it before destroying a
 * stream that ran K-split work, with none of that work captured in a graph that will still be replayed. The stream is
 * synchronised, the buffer freed, and its slot can serve another stream. Without it a buffer lives until the process
 * ends: at most 33 per device (32 streams and the spare), 64 MiB each on a 256-CU part, i.e. up to 2.1 GiB per device for
 * a process that keeps creating streams. No counterpart in the reference. */
int tpamd_scratch_release(void *stream);

/* ------------------------------------------------------------------------------------------------
 * Slicing engine.
 *
 * One job moves a 2-D byte region: `rows` rows of `row_bytes` bytes, row i read at
 * src_dev + i*src_pitch and written at dst_dev + i*dst_pitch. A rank shard of a tensor split on
 * axis d is one such region (rows = prod(shape[:d]), row_bytes = len*prod(shape[d+1:])*itemsize,
 * src_pitch = shape[d]*prod(shape[d+1:])*itemsize); a grouped split is one region per group; the
 * inverse (undo / gather) swaps the roles of the pitches.
 *
 * Replaces, for device-resident tensors, the strided copies behind
 *   Split.__call__ / SplitInChunks.__call__ / SplitInGroupedChunks.__call__
 *     (src/tensor_parallel/state_actions.py:47-48, :76-87, :101-109) followed by `.clone()`
 *     (src/tensor_parallel/shard.py:160), applied to every tensor of a state dict by
 *   process_state_ (src/tensor_parallel/shard.py:132-166) and
 *   convert_state_dict (src/tensor_parallel/dispatch.py:75-131),
 * and their inverses Split.undo / SplitInGroupedChunks.undo (state_actions.py:50-51, :111-119) and
 * the "gather d" concatenation (src/tensor_parallel/cross_device_ops.py:39).
 * ---------------------------------------------------------------------------------------------- */
typedef struct tpamd_copy_job {
    const void *src_dev;
    void *dst_dev;
    uint64_t rows;
    uint64_t row_bytes;
    uint64_t src_pitch; /* bytes between consecutive source rows (ignored when rows == 1) */
    uint64_t dst_pitch; /* bytes between consecutive destination rows */
} tpamd_copy_job;

typedef struct tpamd_copy_plan tpamd_copy_plan; /* opaque: device-resident job table */

/* Validates the jobs, uploads the table (synchronously) and returns a plan that can be run any
 * number of times. Regions of different jobs must not overlap in the destination. Zero-size jobs
 * are legal and skipped. n_jobs == 0 gives a valid empty plan. */
int tpamd_copy_plan_create(const tpamd_copy_job *jobs, size_t n_jobs, tpamd_copy_plan **plan_out);
/* Enqueues the whole plan as ONE kernel launch on `stream`. */
int tpamd_copy_plan_run(const tpamd_copy_plan *plan, void *stream);
/* Bytes read (== bytes written) by one run of the plan. */
uint64_t tpamd_copy_plan_bytes(const tpamd_copy_plan *plan);
int tpamd_copy_plan_destroy(tpamd_copy_plan *plan);

/* The same copies without a plan: up to 16 jobs are passed to the kernel by value, nothing is allocated and
 * nothing has to be kept alive afterwards. For single tensors: one state action on one tensor, the undo of
 * one rule, one "gather d" of W column-parallel outputs. */
int tpamd_copy_jobs_run(const tpamd_copy_job *jobs, size_t n_jobs, void *stream);

/* Transposing mover: for every job, dst[c][r] = src[r][c] over a 2-D region of `rows` x `cols` elements of
 * `elem_bytes` (1, 2 or 4) bytes, staged through LDS in tiles whose rows are whole 128-byte lines on both sides.
 * Weights that the model code keeps as [in, out] and multiplies as x @ w (transformers' Conv1D: GPT-2 c_attn / c_proj /
 * c_fc, sliced by src/tensor_parallel/slicing_configs.py:192-201 and multiplied inside the wrapped module called at
 * src/tensor_parallel/wrapper.py:69-72) are brought into the [out, in] layout of tpamd_linear with it. A job names a
 * region through its base pointer and pitch, so slicing a column or row range out of the unsplit weight and
 * transposing it is one job (a grouped split: one job per group). Up to 16 jobs per call travel in the kernel
 * arguments; nothing is allocated. Pointers and pitches must be multiples of the element size; 16-byte multiples on
 * both sides take the vector path. Source and destination must not overlap. */
typedef struct tpamd_transpose_job {
    const void *src_dev;
    void *dst_dev;
    uint64_t rows;      /* extent of the source region in elements; the destination region is cols x rows */
    uint64_t cols;
    uint64_t src_pitch; /* bytes between consecutive source rows */
    uint64_t dst_pitch; /* bytes between consecutive destination rows */
} tpamd_transpose_job;
int tpamd_transpose_jobs_run(const tpamd_transpose_job *jobs, size_t n_jobs, int elem_bytes, void *stream);

/* Scale state action: out[i] = in[i] / world_size in the tensor's dtype
 * (Scale.__call__, src/tensor_parallel/state_actions.py:59-60). For bf16/f16 the quotient of the
 * fp32-widened value is rounded to nearest even, as torch does. `mul != 0` multiplies instead
 * (Scale.undo, state_actions.py:62-63). */
int tpamd_scale(const void *in_dev, void *out_dev, uint64_t n_elems, int dtype, int world_size, int mul,
                void *stream);

/* ------------------------------------------------------------------------------------------------
 * Partial-sum reduction: out = sum over r < world_size of parts[r], all W partials on this device.
 * Replaces the "sum" output rule of a row-parallel module: AllReduce.__call__
 * (src/tensor_parallel/communications.py:114-116) = ScatterReduce (:119-139) + AllGather (:142-171),
 * whose arithmetic is reduce_add's `sum([...])` (src/tensor_parallel/cross_device_ops.py:43-50).
 * `parts_dev` is a HOST array of `world_size` device pointers (1 <= world_size <= 16); `out_dev`
 * may alias parts_dev[0]. `accum` is a tpamd_accum.
 * ---------------------------------------------------------------------------------------------- */
int tpamd_reduce_partials(const void *const *parts_dev, int world_size, void *out_dev, uint64_t n_elems,
                          int dtype, int accum, void *stream);

/* ------------------------------------------------------------------------------------------------
 * Rank-shard Linears. y[M,N] = act(x[M,K] . w[N,K]^T + bias[N]); fp32 accumulation, one rounding to
 * `dtype` at the store. This is the torch.nn.Linear call made by the wrapped module inside
 * TensorParallelWrapper.forward (src/tensor_parallel/wrapper.py:69-72) on the sliced weight that
 * process_state_ installed (src/tensor_parallel/shard.py:160, features fixed at :184-187):
 *   column-parallel shard: w = rows ts(N,W,r) of the full weight, bias sliced alike;
 *   row-parallel shard:    w = columns ts(K,W,r), x = the matching columns, bias NULL or pre-scaled;
 *                          the result is a partial sum for tpamd_reduce_partials.
 * bias_dev may be NULL. Any shape and alignment is accepted. bf16/f16 operands run on the MFMA kernels
 * when x, w are 16-byte aligned, y and bias 8-byte aligned, K, ldx, ldw are multiples of 8 and N, ldy
 * multiples of 4 (every shape the slicing rules above produce from head-aligned models); other
 * bf16/f16 operands and all fp32 operands run on a scalar-load FMA kernel.
 * ---------------------------------------------------------------------------------------------- */
int tpamd_linear(const void *x_dev, const void *w_dev, const void *bias_dev, void *y_dev, int64_t M, int64_t N,
                 int64_t K, int64_t ldx, int64_t ldw, int64_t ldy, int dtype, int act, void *stream);

/* tpamd_linear followed by one step of the partial-sum reduction, in one launch:
 *   y = round_dtype( round_dtype(act(x . w^T + bias)) + addend ),   addend [M,N] with leading dimension ldadd.
 * With addend = the running sum of the partials of ranks 0..r-1 and (x, w) = rank r's row-parallel shard this is
 * `sum([...])` over the rank partials (src/tensor_parallel/cross_device_ops.py:49, reached from AllReduce.__call__,
 * src/tensor_parallel/communications.py:114-116) taken in rank order, bit for bit: torch adds two same-dtype tensors
 * as the fp32 sum of the widened values, rounded once. F32: y = (x . w^T + bias) + addend in fp32.
 * addend_dev may be y_dev (then ldadd must equal ldy): the partial is accumulated in place. */
int tpamd_linear_add(const void *x_dev, const void *w_dev, const void *bias_dev, const void *addend_dev, void *y_dev,
                     int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldadd, int64_t ldy, int dtype,
                     int act, void *stream);

/* tpamd_linear for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc. It has no counterpart in the reference. Same arguments, same kernels and the same
 * result, bit for bit, as tpamd_linear; the call allocates nothing (no hipMalloc, no hipFree), also at its first use
 * and under stream capture. Where tpamd_linear would put the fp32 partial tiles of a K split into its stream's
 * scratch buffer, this entry point puts them into a fixed array of tpamd_noalloc_scratch_bytes() = 64 MiB that every
 * GPU the library is loaded on holds until the process ends: the size of a stream's buffer on a 256-CU part, so every
 * K split the library picks by itself there fits. A K split that needs more (a part with more CUs, a split forced
 * through the TPAMD_* variables; the message names the size) is refused with TPAMD_ERR_UNSUPPORTED and nothing is
 * launched; tpamd_linear takes such shapes.
 * All calls on one GPU share that GPU's array: calls on the same stream are ordered by it, calls that overlap on
 * different streams of one GPU race on the partial tiles and must be ordered by the caller. */
int tpamd_linear_noalloc(const void *x_dev, const void *w_dev, const void *bias_dev, void *y_dev, int64_t M, int64_t N,
                         int64_t K, int64_t ldx, int64_t ldw, int64_t ldy, int dtype, int act, void *stream);
uint64_t tpamd_noalloc_scratch_bytes(void);

/* h[M,N] = silu(x . wg^T) * (x . wu^T): the gate/up pair of a SiLU-gated MLP shard in one pass over x
 * (two column-parallel torch.nn.Linear calls, a SiLU and a product in the reference's wrapped module;
 * weights sliced by `Split(world_size, dim=0)`, src/tensor_parallel/slicing_configs.py:376-378).
 * The gate and up products are each rounded to `dtype`, then silu and the product are each rounded
 * again, which is what the three separate torch ops of the reference produce. */
int tpamd_swiglu_up(const void *x_dev, const void *wg_dev, const void *wu_dev, void *h_dev, int64_t M, int64_t N,
                    int64_t K, int64_t ldx, int64_t ldw, int64_t ldh, int dtype, void *stream);

/* ------------------------------------------------------------------------------------------------
 * Rank-local attention core: out = softmax(scale * q k^T [+ causal mask]) v over the heads this rank owns.
 * In the reference this is the attention of the wrapped transformers module, run per rank by
 * TensorParallelWrapper.forward (src/tensor_parallel/wrapper.py:69-72) on the rank's share of the heads (head
 * counts divided by the attr rules, e.g. src/tensor_parallel/slicing_configs.py:382-389 for Llama, :414-433 for
 * RefinedWeb/Falcon with grouped key/value heads); the reference itself contains no attention code.
 *   q   [B, Hq, Sq, D], k / v [B, Hkv, Skv, D], out [B, Sq, Hq, D]; Hq a multiple of Hkv (grouped-query: query head h
 *   uses key/value head h / (Hq / Hkv)); D (contiguous) is 64 or 128; dtype BF16 or F16, fp32 accumulation.
 *   strides: 12 element strides, {q batch, q head, q position, k batch, k head, k position, v batch, v head,
 *   v position, out batch, out position, out head}.
 *   causal != 0: query position i sees keys j <= i + (Skv - Sq) (the new tokens are the last Sq positions of the
 *   key range: prefill with Sq == Skv, decode with Sq == 1). No other mask, no dropout.
 * Few rows and many keys (decode) are split over the keys with partials in the per-device scratch buffer
 * described above. Returns TPAMD_ERR_UNSUPPORTED for another head_dim or unaligned rows.
 * ---------------------------------------------------------------------------------------------- */
int tpamd_attention(const void *q_dev, const void *k_dev, const void *v_dev, void *out_dev, int64_t B, int64_t Hq,
                    int64_t Hkv, int64_t Sq, int64_t Skv, int64_t D, const int64_t *strides, float scale, int causal,
                    int dtype, void *stream);

/* Rotary position embedding of the new query / key rows and their hand-over to the rank-local key/value cache, in
 * one launch: the step between a rank shard's QKV projection and tpamd_attention. In the reference the wrapped
 * transformers attention module does this with torch ops on the rank's share of the heads
 * (TensorParallelWrapper.forward, src/tensor_parallel/wrapper.py:69-72; Falcon-40B shard: fused query_key_value split
 * by src/tensor_parallel/slicing_configs.py:430-432, head counts by :455-461), and the cache tensors it returns are
 * routed per rank by select_kv_for_rank / gather_kv (src/tensor_parallel/aux_actions.py:7-15, used at
 * slicing_configs.py:440,446). Here the cache is the rank's own preallocated buffer and the new rows are written in place.
 *   q [B, S, Hq, D], k / v [B, S, Hkv, D]: views of the projection output (any batch / position / head strides, D
 *   contiguous; Hq a multiple of Hkv, and query head h sits at (h / g) * "q group" + (h % g) * "q head" with
 *   g = Hq / Hkv, so a fused output that interleaves each key/value head with its query heads is one view);
 *   cos / sin [B or 1, S, D] in `dtype` (batch stride 0 when shared);
 *   q_out [B, Hq, S, D] receives   q * cos + rotate_half(q) * sin,   rotate_half(x) = cat(-x[D/2:], x[:D/2]);
 *   k_cache / v_cache [B, Hkv, cache_len, D]: positions pos0 .. pos0 + S - 1 receive the rotated k rows and the v rows.
 *   Each of the two products and their sum is rounded to `dtype` (BF16 or F16), which is what the three torch ops of
 *   transformers' apply_rotary_pos_emb produce on tensors of that dtype.
 *   strides: 21 element strides, {q batch, q position, q head, k batch, k position, k head, v batch, v position, v head,
 *   cos/sin batch, cos/sin position, q_out batch, q_out head, q_out position, k_cache batch, k_cache head, k_cache
 *   position, v_cache batch, v_cache head, v_cache position, q group (= g * q head for a plain [B, S, Hq, D] view)}; all
 *   multiples of 8, all pointers 16-byte aligned.
 * D is 64 or 128 and the whole head is rotated (TPAMD_ERR_UNSUPPORTED otherwise). q_out may not overlap q. */
int tpamd_rope_append(const void *q_dev, const void *k_dev, const void *v_dev, const void *cos_dev, const void *sin_dev,
                      void *q_out_dev, void *k_cache_dev, void *v_cache_dev, int64_t B, int64_t S, int64_t Hq, int64_t Hkv,
                      int64_t D, int64_t pos0, int64_t cache_len, const int64_t *strides, int dtype, void *stream);

/* Decode step of the same call site with tpamd_rope_append and tpamd_attention in one: one new position per sequence
 * on a rank-local cache that holds pos0 positions (reference: the wrapped attention module's torch ops, as for the two
 * entry points above; src/tensor_parallel/wrapper.py:69-72, aux_actions.py:7-15, slicing_configs.py:430-461).
 *   q [B, Hq, D], k / v [B, Hkv, D]: the new position's raw rows, views of the projection output (query head h at
 *   (h / g) * "q group" + (h % g) * "q head", g = Hq / Hkv); cos / sin [B or 1, D];
 *   k_cache / v_cache [B, Hkv, cache_len, D]: positions 0 .. pos0 - 1 are read, position pos0 receives the rotated key
 *   and the value (the same bits tpamd_rope_append writes);
 *   out [B, Hq, D] = softmax(scale * rot(q) . [cache keys, rot(k)]^T) [cache values, v].
 * Two launches instead of three: the attention kernel rotates its query fragments itself and leaves one partial result
 * per key range of the cache; the merge adds the new position (its score in fp32 from the rotated rows) and writes the
 * cache rows. Rounding differs from the two-call sequence only in that the new position's probability is not rounded to
 * `dtype` before it weighs its value.
 *   strides: 16 element strides, {q batch, q head, q group, k batch, k head, v batch, v head, cos/sin batch (0 when
 *   shared), k_cache batch, k_cache head, k_cache position, v_cache batch, v_cache head, v_cache position, out batch,
 *   out head}; the first 14 multiples of 8, the last two of 4; pointers 16-byte aligned (out: 8).
 * Needs the stream's scratch buffer for the partial results: TPAMD_ERR_UNSUPPORTED when there is none (the stream's
 * first use of it under capture, or a batch too large for it); callers then use the two entry points above. */
int tpamd_attention_decode_rope(const void *q_dev, const void *k_dev, const void *v_dev, const void *cos_dev,
                                const void *sin_dev, void *k_cache_dev, void *v_cache_dev, void *out_dev, int64_t B,
                                int64_t Hq, int64_t Hkv, int64_t D, int64_t pos0, int64_t cache_len, const int64_t *strides,
                                float scale, int dtype, void *stream);

/* tpamd_attention_decode_rope with the number of cached positions read on the device: *pos_dev (int64, device memory, 8-byte
 * aligned) is read by the kernels when they run, not by this call, so a HIP graph that holds the call serves every decode
 * step (the caller adds 1 to *pos_dev after each step, on the same stream). No counterpart in the reference, whose
 * forwards are Python (src/tensor_parallel/tensor_parallel.py:139-161); transformers' StaticLayer keeps this count on the
 * device as `cumulative_length`. The launches are laid out for `cache_len` positions (the capacity of the caches) and the
 * blocks share out the positions there are; a count outside [0, cache_len) leaves the caches unwritten. Same arguments,
 * requirements and errors otherwise. */
int tpamd_attention_decode_rope_devpos(const void *q_dev, const void *k_dev, const void *v_dev, const void *cos_dev,
                                       const void *sin_dev, void *k_cache_dev, void *v_cache_dev, void *out_dev, int64_t B,
                                       int64_t Hq, int64_t Hkv, int64_t D, const int64_t *pos_dev, int64_t cache_len,
                                       const int64_t *strides, float scale, int dtype, void *stream);

/* Weight-only int8 shard Linear with fp16/bf16 outlier columns:
 *   y[m,n] = act( scale[n] * sum_k x[m,k]*wq[n,k]  +  sum_j x[m,outlier_idx[j]] * w_out[n,j]  + bias[n] )
 * wq is int8 [N,K] (zero in the outlier columns), scale fp32 [N], outlier_idx int32 [n_out] (sorted,
 * distinct, < K), w_out [N,n_out] in `dtype` with leading dimension ld_wout. Not part of the reference
 * (its README points to LLM.int8 notebooks); defined here in closed form.
 * Up to 64 rows the weights are streamed once (HBM-bound kernels); up to 128-256 rows once per slab of 64 rows; above
 * that they go through the matrix pipe once, converted to `dtype` (exactly) on their way into LDS.
 * Requirements: dtype is F16 or BF16; K % 16 == 0; ldw (int8 elements) % 16 == 0. */
int tpamd_linear_w8(const void *x_dev, const void *wq_dev, const void *scale_dev, const void *outlier_idx_dev,
                    const void *w_out_dev, int64_t n_out, const void *bias_dev, void *y_dev, int64_t M, int64_t N,
                    int64_t K, int64_t ldx, int64_t ldw, int64_t ld_wout, int64_t ldy, int dtype, int act,
                    void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TPAMD_H */
