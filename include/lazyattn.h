/* lazyattn.h -- C ABI of the MI355X (gfx950) deferred-RoPE prefix-prefill library.
 *
 * Plain pointers and sizes only; every pointer that is dereferenced on the GPU is a
 * device pointer.  No entry point allocates, frees, synchronises or throws: each
 * returns 0 or a negative LAZYATTN_E_* code and enqueues its work on the given HIP
 * stream.  Paths in the comments are relative to the reference checkout.
 */
#ifndef LAZYATTN_H
#define LAZYATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types */
enum {
    LAZYATTN_F32 = 0,
    LAZYATTN_BF16 = 1,
    LAZYATTN_F16 = 2,
    LAZYATTN_FP8_E4M3 = 3, /* OCP e4m3fn, cache only */
    LAZYATTN_FP8_E5M2 = 4  /* cache only */
};

/* how the rotation position of a cached key is derived */
enum {
    LAZYATTN_POS_NATURAL = 0,      /* p = n                      old_ops/prefix_prefill.py:183-184 */
    LAZYATTN_POS_OFFSET = 1,       /* p = q_offset-1+o | n       old_ops/prefix_prefill.py:186-191 */
    LAZYATTN_POS_BLOCK_UNIFORM = 2 /* p = q_offset-1 | 0 (page)  ops/prefix_prefill.py:180-186     */
};

/* kernel selection */
enum {
    LAZYATTN_KERNEL_AUTO = 0,
    LAZYATTN_KERNEL_GENERIC = 1, /* fp32 arithmetic, any geometry */
    LAZYATTN_KERNEL_MFMA = 2,    /* bf16 / fp16 MFMA, head_dim 128, 64 or a multiple of 16 below 128, pages of 16 or 32 slots; workgroup shape chosen */
    LAZYATTN_KERNEL_MFMA4 = 3,   /* ... with 4 x 32 query rows per workgroup */
    LAZYATTN_KERNEL_MFMA8 = 4    /* ... with 8 x 32 query rows per workgroup */
};

/* which launches of a call to enqueue (profiling aid; default = both) */
enum { LAZYATTN_PHASE_MAIN = 1, LAZYATTN_PHASE_COMBINE = 2, LAZYATTN_PHASE_ALL = 3 };

enum {
    LAZYATTN_OK = 0,
    LAZYATTN_E_NULL = -1,        /* a required pointer is null */
    LAZYATTN_E_SHAPE = -2,       /* inconsistent sizes (heads, head_dim, x, block_size ...) */
    LAZYATTN_E_DTYPE = -3,       /* unsupported type combination */
    LAZYATTN_E_UNSUPPORTED = -4, /* valid request the selected kernel cannot run */
    LAZYATTN_E_WORKSPACE = -5,   /* workspace missing or too small */
    LAZYATTN_E_LAUNCH = -6,      /* hipLaunchKernel failed */
    LAZYATTN_E_SCRATCH_LIMIT = -7 /* lazyattn_prefix_prefill_static_scratch: the call needs more than the static buffer holds */
};

/* Arguments of one prefix-prefill call.  Replaces the Triton launch in
 *   lazy_attn/lazy/attention/old_ops/prefix_prefill.py:491-554  (un-rotated cache)
 *   lazy_attn/lazy/attention/ops/prefix_prefill.py:681-743      (block-uniform rotation)
 * with the same operands.  Strides are in ELEMENTS.  q_offset / q_mask carry their
 * own strides (the reference indexes them with the block table's strides,
 * ops/prefix_prefill.py:180-182,267-268 -- pass the same values to get that).  */
typedef struct lazyattn_prefill_params {
    const void *q;       /* [T, Hq, D]   already rotated by the caller */
    const void *k;       /* [T, Hkv, D]  new-token keys */
    const void *v;       /* [T, Hkv, D] */
    void *o;             /* [T, Hq, D]   written in place, rows t >= q_len untouched */
    const void *k_cache; /* [NB, Hkv, D/x, BS, x] */
    const void *v_cache; /* [NB, Hkv, D, BS] */
    const int32_t *block_table; /* [B, NBmax] */
    const int32_t *q_offset;    /* [B, NBmax] or NULL (= zeros) */
    const int32_t *q_mask;      /* [B, NBmax] or NULL (= zeros) */
    const uint8_t *is_lazy;     /* [B] bytes or NULL (= all set); only read for
                                   LAZYATTN_POS_BLOCK_UNIFORM (ops/prefix_prefill.py:98) */
    const void *b_start_loc;    /* [B+1] int32 or int64, see index_bits */
    const void *b_seq_len;      /* [B] */
    const void *cos_sin_cache;  /* [max_pos, rotary_dim]: row p = cos(p*inv) | sin(p*inv); rows are read
                                   for the 16-slot runs that hold real keys and for the new tokens
                                   (LAZYATTN_POS_NATURAL: max_pos >= the longest context rounded up to
                                   16 and >= the longest b_seq_len), like the reference's kernels */
    const void *cos_sin_packed; /* optional: the same table re-laid out by lazyattn_pack_cos_sin_cache()
                                   as [2][rotary_dim/16][packed_rows][8], so that the 16 slots of a page
                                   read 16 consecutive 16-byte chunks; NULL = read the row-major table */
    const float *k_scale;       /* 1 element, read only for fp8 caches: key = fp8 value * k_scale (old_ops/prefix_prefill.py:239-241). */
    const float *v_scale;       /* The matrix-core kernel with bf16 operands applies the two scales to Q and to the final 1/l
                                   instead of to every cached element (linear, so the same result up to the one rounding of
                                   the scaled element the reference makes; identical for power-of-two scales). */
    void *workspace;            /* split-KV partials; lazyattn_prefill_workspace_bytes() */
    int64_t workspace_bytes;

    int64_t q_stride[3], k_stride[3], v_stride[3], o_stride[3];
    int64_t kc_stride[5], vc_stride[4];
    int64_t bt_stride[2], qo_stride[2], qm_stride[2];
    int64_t table_stride;       /* row stride of cos_sin_cache */

    int32_t batch, num_q_heads, num_kv_heads, head_dim;
    int32_t block_size, x;      /* x = k_cache.shape[4] */
    int32_t max_q_len;          /* max_input_len: sizes the grid (ops/prefix_prefill.py:681-682) */
    int32_t rotary_dim;         /* must equal head_dim (the reference assumes it too) */
    int32_t sliding_window;     /* <= 0 disables */
    int32_t dtype;              /* q/k/v/o element type */
    int32_t cache_dtype;        /* dtype, or FP8_* */
    int32_t table_dtype;        /* dtype or F32 */
    int32_t index_bits;         /* 32 or 64: b_start_loc / b_seq_len */
    int32_t pos_mode;           /* LAZYATTN_POS_* */
    int32_t rotate_new_k;       /* 1: rotate new-token K at ctx_len+m (old_ops:342-362) */
    int32_t skip_decode;        /* 1: requests with q_len == 1 are not written (old_ops:109-110) */
    int32_t fp32_rotary;        /* FORCE_FP32_ROTARY (old_ops:248-254); the MFMA kernel always
                                   rotates in fp32 and rounds once */
    int32_t kernel;             /* LAZYATTN_KERNEL_* */
    int32_t num_splits;         /* key-axis splits of every request; 0 = choose: for one request on the host, for a
                                   batch of up to 256 requests per request on the device, from the lengths */
    int32_t phases;             /* LAZYATTN_PHASE_*; 0 = all */
    float sm_scale;
    int32_t num_tokens;         /* rows of `o` (>= b_start_loc[B]); sizes the split-KV workspace */
    int32_t max_seq_len;        /* upper bound of b_seq_len, 0 = unknown; only steers the split count */
    int32_t packed_rows;        /* rows of cos_sin_packed (0 when it is NULL) */
    /* ---- read by lazyattn_paged_decode_rotary() only ---- */
    const int64_t *packed_block_table; /* optional [B, NBmax]: [block:32 | q_offset:16 | q_mask:16] per entry, the table
                                   the reference's q_len==1 kernel walks (ops/models/llama_v1.py:157-160,
                                   ops/chunked_prefill_paged_decode.py:162-164).  When set it replaces block_table,
                                   q_offset and q_mask (which may then be NULL): one 8-byte read per page. */
    int64_t pbt_stride[2];
    const float *rope_freqs;    /* optional [rotary_dim/2] float32 inverse frequencies, radians per position
                                   (rope_freqs, model_executor/rope/cos_sin.py:24-59).  When set, cos/sin are computed
                                   in the kernel (rope_cos_sin_from_freqs, :62-66; the reference's COMPUTE_COS_SIN
                                   switch, ops/chunked_prefill_paged_decode.py:146-151) and cos_sin_cache is not read. */
} lazyattn_prefill_params;

/* Bytes of workspace lazyattn_prefix_prefill() may need for these sizes (0 when the
 * chosen kernel writes `o` directly: one request that is not split, or num_splits = 1).  A call with several
 * requests and num_splits = 0 always needs it: which requests are split is decided on the device.  The workspace
 * holds partial rows (and, for batches, a 16-byte record per request at its head); nothing in it has to be
 * initialised, and a call reads only what the same call wrote.  Pure host arithmetic.  No reference
 * counterpart: Triton's launch has no split-KV. */
size_t lazyattn_prefill_workspace_bytes(const lazyattn_prefill_params *p);

/* Deferred-RoPE prefix-prefill attention.  Replaces `_fwd_kernel[grid](...)`
 * (old_ops/prefix_prefill.py:493, ops/prefix_prefill.py:683). `stream` is a hipStream_t. */
int lazyattn_prefix_prefill(const lazyattn_prefill_params *p, void *stream);

/* lazyattn_prefix_prefill() for callers that cannot allocate device memory or hand over a workspace: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the
 * reference.  Same arguments and results; `workspace` / `workspace_bytes` are ignored and the split-KV
 * partials go to a buffer of lazyattn_static_scratch_bytes() (32 MiB) that the library holds statically in
 * each GPU's memory until the process ends.  A call that would need more returns
 * LAZYATTN_E_SCRATCH_LIMIT (lazyattn_prefill_workspace_bytes() tells beforehand).  Allocates nothing.  All
 * calls on one GPU share that buffer: calls that overlap in time on one GPU (two streams) race; calls on one
 * stream, or otherwise ordered, are safe -- every partial a call merges was written by that call.
 * The first use on a GPU looks the buffer's address up (which may load the library's code onto that GPU):
 * call lazyattn_static_scratch_prepare() -- or make one call -- with that GPU current before entering a region
 * that must not allocate, such as a stream capture. */
int lazyattn_prefix_prefill_static_scratch(const lazyattn_prefill_params *p, void *stream);
size_t lazyattn_static_scratch_bytes(void);
int lazyattn_static_scratch_prepare(void);

/* Which kernel lazyattn_prefix_prefill() launches for these arguments: LAZYATTN_KERNEL_GENERIC, LAZYATTN_KERNEL_MFMA4
 * or LAZYATTN_KERNEL_MFMA8 (a negative LAZYATTN_E_* code when the call would be refused).  *num_splits (optional)
 * receives the number of key-axis splits; *reason (optional) a static string saying why the fp32 kernel -- some
 * hundred times slower than the matrix-core kernels -- is the one, NULL otherwise.  Pure host arithmetic.  No
 * reference counterpart (Triton has one kernel); for callers who want to see the fallback before they pay for it. */
int lazyattn_prefill_kernel_for(const lazyattn_prefill_params *p, int32_t *num_splits, const char **reason);
/* The same for lazyattn_paged_decode_rotary(): LAZYATTN_KERNEL_MFMA (the streaming kernel, the only one that reads
 * packed_block_table / rope_freqs), LAZYATTN_KERNEL_GENERIC, or the LAZYATTN_E_* code the call would return. */
int lazyattn_paged_decode_kernel_for(const lazyattn_prefill_params *p);

/* q_len == 1 rows: every key (the new token included) comes from the paged cache.
 * pos_mode NATURAL: each key is rotated at its natural position; replaces
 *   `kernel_paged_attention_2d[(num_seqs, num_kv_heads)](...)`
 *   (old_ops/chunked_prefill_paged_decode.py:396-442).
 * pos_mode BLOCK_UNIFORM: each page of a lazy request is rotated forward by q_offset-1
 *   (the reference de-rotates Q by the same angle instead, which gives the same scores);
 *   other requests are not rotated; replaces `kernel_paged_attention_2d_llama`
 *   (ops/models/llama_v1.py:91-288, launched at ops/chunked_prefill_paged_decode.py:171-221).
 * Uses the same struct: k, v, rotate_new_k are ignored; requests with q_len != 1 are
 * skipped (old_ops/chunked_prefill_paged_decode.py:72-79). */
int lazyattn_paged_decode_rotary(const lazyattn_prefill_params *p, void *stream);

/* Bytes of workspace lazyattn_paged_decode_rotary() can use for these sizes: partials of the
 * slices one request's pages are cut into so that few requests still fill the GPU (0 = none).
 * Without (enough) workspace the call runs unsliced.  Pure host arithmetic; no reference
 * counterpart (the Triton kernel is one program per (sequence, kv head)). */
size_t lazyattn_paged_decode_workspace_bytes(const lazyattn_prefill_params *p);

/* ---- the step before the attention call: rotary embedding of the new tokens + paged-cache write ----
 * One launch does what the reference does with two third-party ops per layer:
 *   rotary_embedding(positions, query, key_or_None, head_size, cos_sin_cache, is_neox)
 *     (lazy_attn/lazy/model_executor/layers/rotary_embedding.py:67-94: query only under the
 *      un-rotated-cache variant, query and key otherwise, :48-49), in place, NeoX pairing (d, d + R/2);
 *   PagedAttention.write_to_paged_cache(key, value, key_cache, value_cache, slot_mapping,
 *     kv_cache_dtype, k_scale, v_scale)  (lazy_attn/lazy/attention/backends/triton_attn.py:100-109):
 *     token t -> slot_mapping[t] = block * block_size + offset (negative: not written);
 *     fp8 caches store value / scale (a true division), saturated to +-448 and rounded to e4m3, or to +-57344 and
 *     e5m2; NaN stays NaN.  An fp8 K cache needs x % 8 == 0.
 * The key written to the cache is the key as it is left in `k` (rotated iff rotate_k). */
typedef struct lazyattn_rope_write_params {
    void *q;                    /* [T, Hq, D], rotated in place when rotate_q; may be NULL when !rotate_q */
    void *k;                    /* [T, Hkv, D], rotated in place when rotate_k */
    const void *v;              /* [T, Hkv, D] */
    void *k_cache;              /* [NB, Hkv, D/x, BS, x]; NULL = no cache write */
    void *v_cache;              /* [NB, Hkv, D, BS] */
    const void *slot_mapping;   /* [T] int32 or int64 (slot_bits); NULL = no cache write */
    const void *positions;      /* [T] int32 or int64 (pos_bits): rows of the cos/sin table */
    const void *cos_sin_cache;  /* [max_pos, rotary_dim] */
    const float *k_scale;       /* 1 element each, read only for fp8 caches */
    const float *v_scale;
    int64_t q_stride[3], k_stride[3], v_stride[3];   /* in elements */
    int64_t kc_stride[5], vc_stride[4];
    int64_t table_stride;
    int32_t num_tokens, num_q_heads, num_kv_heads, head_dim, rotary_dim, block_size, x;
    int32_t dtype;              /* q/k/v: LAZYATTN_F32 / BF16 / F16 */
    int32_t cache_dtype;        /* = dtype, or LAZYATTN_FP8_E4M3 / LAZYATTN_FP8_E5M2 */
    int32_t table_dtype;        /* = dtype, or LAZYATTN_F32 */
    int32_t rotate_q, rotate_k;
    int32_t pos_bits, slot_bits;
} lazyattn_rope_write_params;

int lazyattn_rope_and_cache_write(const lazyattn_rope_write_params *p, void *stream);

/* Per-page rotation metadata of a batch, written on the device into the [batch, row_len] int32
 * buffers the attention kernels read.  Same integers as metadata_for_lazy_attention /
 * metadata_for_mepic (lazy_attn/lazy/core/sched/scheduler.py:758-787); replaces the per-request host
 * loop and the two host-to-device copies of lazy_attn/lazy/worker/gpu_model_runner.py:193-239.
 * Documents in CSR form: request b owns doc_lens[doc_start[b] .. doc_start[b+1]) (true lengths) and
 * the matching doc_lens_padded (multiples of block_size).  zero_offsets = the un-rotated-cache
 * variant (all q_offset 0).  Rows are written completely (zeros beyond the query page).
 * max_offset (optional, [batch]) receives each request's largest offset value, for the
 * 16-bit admission check of the packed block table (worker/gpu_model_runner.py:212-226). */
int lazyattn_build_rotation_metadata(const int32_t *doc_lens, const int32_t *doc_lens_padded,
                                     const int32_t *doc_start, int32_t batch, int32_t block_size,
                                     int32_t zero_offsets, int32_t *q_offset, int32_t *q_mask,
                                     int64_t row_stride, int32_t row_len, int32_t *max_offset, void *stream);

/* Packed block table of the block-uniform decode path, [block:32 | q_offset:16 | q_mask:16] per int64
 * entry (layout of lazy_attn/lazy/attention/ops/models/llama_v1.py:157-160), for the listed rows
 * (rows == NULL: rows 0 .. n_rows-1), in one launch.  Replaces the tensor-op sequence of
 * _rebuild_packed_block_table (lazy_attn/lazy/worker/gpu_model_runner.py:296-340), full or delta. */
int lazyattn_pack_block_table(const int32_t *block_table, int64_t bt_stride, const int32_t *q_offset,
                              const int32_t *q_mask, int64_t row_stride, const int32_t *rows, int32_t n_rows,
                              int32_t row_len, int64_t *packed, int64_t packed_stride, void *stream);

/* Copy-and-re-rotate of cached document blocks, all blocks of one layer in one launch.
 * Replaces the per-layer, per-block eager loop of block_attn_vllm/gpu_model_runner.py:94-106 over
 * copy_paged_block + place_paged_block_keys (block_attn_vllm/utils.py:48-95).
 * items: [num_items][4] int32 on the device = (new_id, old_id, from_start, to_start): block old_id
 * (K and V) is copied to new_id, and slot o of the K copy goes from rotation position from_start + o to
 * to_start + o (un-rotate, then rotate, NeoX pairing, rows of cos_sin_cache).  new_id == old_id re-rotates
 * in place.  The new blocks must be distinct from each other and from every old block of the call. */
typedef struct lazyattn_reposition_params {
    void *k_cache;              /* [NB, Hkv, D/x, BS, x] */
    void *v_cache;              /* [NB, Hkv, D, BS] */
    const int32_t *items;
    const void *cos_sin_cache;  /* [max_pos, D] */
    int64_t kc_stride[5], vc_stride[4];
    int64_t table_stride;
    int32_t num_items, num_kv_heads, head_dim, block_size, x;
    int32_t dtype;              /* cache element type: LAZYATTN_F32 / BF16 / F16 */
    int32_t table_dtype;        /* = dtype, or LAZYATTN_F32 */
} lazyattn_reposition_params;

int lazyattn_reposition_blocks(const lazyattn_reposition_params *p, void *stream);

/* cos/sin table builder on the device: out[p, i] = cos(p*inv[i]), out[p, R/2+i] = sin(..),
 * inv = base^(-2i/R), optionally Llama-3 smoothed.  Restates
 * lazy_attn/lazy/model_executor/rope/cos_sin.py:24-66 and the third-party table layout
 * the kernels read (old_ops/prefix_prefill.py:192-193,231-232).  rope_type 0 = plain,
 * 1 = Llama-3.  Angles are formed in float64 so rows at positions beyond 2^16 keep
 * full float32 accuracy. */
int lazyattn_build_cos_sin_cache(void *out, int32_t out_dtype, int64_t row_stride,
                                 int32_t max_position, int32_t rotary_dim, double base,
                                 int32_t rope_type, double scaling_factor,
                                 double low_freq_factor, double high_freq_factor,
                                 int32_t orig_max_position, void *stream);

/* Re-layout of a cos/sin table for the MFMA kernel's per-token gather:
 * packed[h][c][p][e] = table[p, h*R/2 + c*8 + e]  (h = 0 cos, 1 sin; c < R/16; e < 8).
 * `packed` holds rows * rotary_dim elements of the table's type.  Done once per table
 * (the table is a model constant); no reference counterpart. */
int lazyattn_pack_cos_sin_cache(const void *table, void *packed, int32_t dtype, int64_t row_stride,
                                int32_t rows, int32_t rotary_dim, void *stream);

const char *lazyattn_error_string(int code);
int lazyattn_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* LAZYATTN_H */
