/*
 * alignedkv.h -- C ABI of the MI355X (gfx950) AlignedKV library, libalignedkv_hip.so.
 *
 * The five akv_* ops below are what the reference's Python layer binds through pybind11 as
 * `cuda_module` (reference: extension/csrc/KV_cache_ops.cpp:69-75, loaded by
 * extension/KV_cache_cpp_extention.py:6-9).  Every argument that the reference passes as a
 * torch.uint8 tensor is a plain device pointer here; outputs the reference allocates with
 * torch::empty are caller-allocated.  Scalar arguments keep the reference's names, order and meaning.
 *
 * Conventions
 *   - all pointers are device pointers on the current HIP device; `stream` is a hipStream_t
 *     (NULL = the default stream); every call is asynchronous on that stream;
 *   - fp16 tensors are passed as bytes (little endian halves), as in the reference;
 *   - return value 0 = launched; non-zero = rejected, nothing was launched and
 *     akv_last_error() returns a description (thread local);
 *   - plane layouts (extension/k_cache_file.py:45-53, extension/v_cache_file.py:46-54):
 *       K first_8 [bsz, n_kv_heads, n_max_blocks, d_head, d_block]      uint8
 *       K mid_4 / last_4 [bsz, n_kv_heads, n_max_blocks, d_head, d_block/2]  two slots per byte,
 *                                                                      even slot in the high nibble
 *       V first_8 [bsz, n_kv_heads, max_seq_len, head_dim]             uint8
 *       V mid_4 / last_4 [bsz, n_kv_heads, max_seq_len, head_dim/2]    even channel in the high nibble
 *   - fetch levels: 0 = all planes, 1 = last_4 not fetched (replaced by 0x8), 2 = mid_4 and
 *     last_4 not fetched (low byte replaced by 0x80).
 */
#ifndef ALIGNEDKV_H
#define ALIGNEDKV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *akv_stream_t; /* hipStream_t */

#if defined(__GNUC__)
#define AKV_API __attribute__((visibility("default")))
#else
#define AKV_API
#endif

#define AKV_OK 0
#define AKV_ERR_INVALID 1     /* bad argument (null pointer, unsupported shape, size mismatch) */
#define AKV_ERR_LAUNCH 2      /* the HIP runtime refused the launch */

/* Library version (major*100 + minor). */
AKV_API int akv_version(void);

/* Description of the last non-zero return on this thread ("" if none). */
AKV_API const char *akv_last_error(void);

/*
 * Replaces k_cache_save (reference: extension/csrc/KV_cache_ops.cpp:5-16, extension/csrc/K_cache.cu:97-164).
 * k_new: fp16 [bsz, seqlen, n_kv_heads, d_head] contiguous.
 * start_pos == 0 or seqlen % d_block == 0: writes blocks start_pos/d_block .. +n_blocks from tokens
 * 0 .. min(n_blocks*d_block, seqlen) of k_new.  Otherwise, seqlen == 1: inserts one token at slot
 * start_pos % d_block of block start_pos / d_block.  Nibble bytes are written, not accumulated
 * (identical to the reference's `+=` on zero-initialised planes).  Needs d_block % 8 == 0, d_head % 2 == 0.
 * Beyond the reference (which launches nothing for it): start_pos != 0, seqlen % d_block != 0, with d_block,
 * start_pos and seqlen multiples of 64 -- whole 64-token tiles appended inside a block, the result of seqlen
 * single-token inserts.  Used by caches whose K planes have 256-token blocks and a 64-token rest buffer.
 */
AKV_API int akv_k_cache_save(uint8_t *first_8, uint8_t *mid_4, uint8_t *last_4, const uint8_t *k_new,
                     int bsz, int n_kv_heads, int n_blocks, int n_max_blocks, int d_head, int d_block,
                     int start_pos, int seqlen, akv_stream_t stream);

/*
 * Replaces k_cache_compute (reference: extension/csrc/KV_cache_ops.cpp:18-32, extension/csrc/K_cache.cu:314-395).
 * k_column_max_multiply_q: uint8 [bsz, 1, n_kv_heads, d_head]; k_column_max_multiply_q_max: uint8
 * [bsz, 1, n_kv_heads, 1]; q: fp16 [bsz, 1, n_kv_heads, d_head].
 * s_out: fp16 [bsz, n_kv_heads, 1, (n_blocks+1)*d_block] (the tensor the reference returns); entries
 * < n_blocks*d_block are written, the last d_block entries of every row are left untouched.
 * s[b,h,t] = fp16( (sum_d khat[t,d]*q[d]) * half(sqrt_dim) ), fp32 accumulation.  `sqrt_dim` is the
 * reciprocal 1/sqrt(d_head) as in the reference.  `seqlen` is accepted for signature parity and unused.
 * levels_out (optional, may be NULL): uint8 [bsz, n_kv_heads, d_head], the fetch level each channel used.
 */
AKV_API int akv_k_cache_compute(const uint8_t *first_8, const uint8_t *mid_4, const uint8_t *last_4,
                        const uint8_t *k_column_max_multiply_q, const uint8_t *k_column_max_multiply_q_max,
                        const uint8_t *q, uint8_t *s_out, uint8_t *levels_out,
                        int bsz, int n_kv_heads, int n_blocks, int n_max_blocks, int d_head, int d_block,
                        int seqlen, float sqrt_dim, int reference, akv_stream_t stream);

/*
 * Replaces v_cache_save (reference: extension/csrc/KV_cache_ops.cpp:34-43, extension/csrc/V_cache.cu:44-80).
 * v_new: fp16 [bsz, v_new_seq, n_local_kv_heads, head_dim] contiguous (v_new_seq = v_new.size(1) in the
 * reference); its first seq_len tokens are stored at rows start_pos .. start_pos+seq_len.
 */
AKV_API int akv_v_cache_save(uint8_t *first_8, uint8_t *mid_4, uint8_t *last_4, const uint8_t *v_new,
                     int bsz, int n_local_kv_heads, int max_seq_len, int head_dim, int start_pos,
                     int seq_len, int v_new_seq, akv_stream_t stream);

/*
 * Replaces v_cache_test_compute (reference: extension/csrc/KV_cache_ops.cpp:45-54, extension/csrc/V_cache.cu:125-168).
 * test_s_value: fp16 [bsz, heads, 1, top_max_k]; test_s_index: int32 [bsz, heads, 1, top_max_k];
 * test_o_out: fp16 [bsz, heads, 1, head_dim].
 * test_o[b,h,d] = fp16( sum_i s_i * |fp16(first_8[b,h,idx_i*top_max_k+i,d]<<8 | 0x80)| ).
 * Token indices must lie in [0, max_seq_len).
 */
AKV_API int akv_v_cache_test_compute(const uint8_t *first_8, const uint8_t *mid_4, const uint8_t *last_4,
                             const uint8_t *test_s_value, const uint8_t *test_s_index, uint8_t *test_o_out,
                             int bsz, int n_local_kv_heads, int max_seq_len, int head_dim, int top_max_k,
                             akv_stream_t stream);

/* Bytes of device scratch akv_v_cache_compute needs for this shape (split-sequence partial sums). */
AKV_API size_t akv_v_cache_compute_workspace_bytes(int bsz, int n_local_kv_heads, int head_dim, int n_tokens);

/*
 * Replaces v_cache_compute (reference: extension/csrc/KV_cache_ops.cpp:56-67, extension/csrc/V_cache.cu:310-374).
 * s: fp16, row (b,h) starts at element (b*heads + h)*s_last_dim; s_exp_expect_alignment_min: uint8, entry
 * b*heads + h is used; o_out: fp16 [bsz, heads, 1, head_dim].
 * o[b,h,d] = fp16( sum_{t < start_pos_add_seqlen} vhat[t,d]*s[t] ), fp32 accumulation.
 * levels_out (optional): uint8 [bsz, heads, start_pos_add_seqlen], the fetch level each token used.
 * workspace: >= akv_v_cache_compute_workspace_bytes(...) bytes, 256-byte aligned, private to this call
 * until the stream has passed it.
 */
AKV_API int akv_v_cache_compute(const uint8_t *first_8, const uint8_t *mid_4, const uint8_t *last_4,
                        const uint8_t *s, const uint8_t *s_exp_expect_alignment_min, uint8_t *o_out,
                        uint8_t *levels_out, void *workspace, size_t workspace_bytes,
                        int bsz, int n_local_kv_heads, int max_seq_len, int head_dim, int s_last_dim,
                        int start_pos_add_seqlen, int reference, akv_stream_t stream);

/*
 * Fused decode step for one layer: appends one token per sequence and attends over the whole cache.
 * Replaces, in one call, what the reference does in Python around its three compute ops:
 * QuantizedCache_AlignedKV.decoding (model/KVCache_AlignedKV.py:116-124), K_Cache_Class.save /
 * decoding_compute (extension/k_cache_file.py:97-118,132-159) and V_Cache_Class.save / test_compute /
 * decoding_compute (extension/v_cache_file.py:97-116,119-190), with the same arithmetic and order:
 * column-max update, rest-buffer append (flush of a full 64-token buffer into the planes first), plane
 * scores with per-channel fetch levels, fp16 tail scores, optional additive fp16 mask, fp32 softmax to
 * fp16 probabilities, 32-bucket arg-max probe, alignment threshold, plane output with per-token fetch
 * levels, fp16 tail output.
 *
 * State, updated in place: K/V planes; k_/v_exp_column_max uint8 [bsz,1,heads,head_dim]; restk/restv fp16
 * [bsz, d_block, heads, head_dim].  The caller keeps the three counters and advances them after the call:
 * cur_len += 1; rest_len += 1; if rest_len == d_block: rest_start += d_block, rest_len = 0.
 * q, k_new, v_new, out: fp16 [bsz,1,heads,head_dim].  mask: optional fp16 [bsz, >= cur_len+1] with row
 * stride mask_stride (halves; 0 = one row shared by all sequences), added to the scores of every head.
 * scores / probs: fp16 [bsz, heads, row_stride] scratch that also serves as debug output (scores of the
 * flushed blocks and the tail before the mask; probabilities of tokens < cur_len+1); row_stride % 8 == 0,
 * row_stride >= flushed tokens + d_block.
 * k_levels_out uint8 [bsz,heads,head_dim], v_levels_out uint8 [bsz,heads,flushed tokens], amin_out uint8
 * [bsz,heads]: optional (NULL) records of the fetch decisions.
 * flags: AKV_STEP_LITERAL_BROADCAST reproduces the reference's threshold indexing as written
 * (extension/v_cache_file.py:157-160 broadcasts [B,H,1,D] against [B,1,H,D]); AKV_STEP_NO_PROBS_RECORD lets the step
 * leave `probs` unwritten where no kernel of the step reads it back (the form of the step that keeps a row's
 * probabilities on chip: 2 MB of stores, 0.7 us, at batch 8 x 32 heads x 4096 tokens) -- `probs` is still required,
 * the other forms use it as scratch, and its contents are then unspecified.
 * Supported: head_dim 64/128/256, d_block 64, top_max_k 32; other shapes go through the five ops.
 */
#define AKV_STEP_LITERAL_BROADCAST 1
#define AKV_STEP_NO_PROBS_RECORD 2
AKV_API size_t akv_decode_step_workspace_bytes(int bsz, int n_q_heads, int head_dim, int max_seq_len);
AKV_API int akv_decode_step(uint8_t *k_first_8, uint8_t *k_mid_4, uint8_t *k_last_4, uint8_t *v_first_8,
                            uint8_t *v_mid_4, uint8_t *v_last_4, uint8_t *k_exp_column_max,
                            uint8_t *v_exp_column_max, uint8_t *restk, uint8_t *restv, const uint8_t *q,
                            const uint8_t *k_new, const uint8_t *v_new, const uint8_t *mask, int mask_stride,
                            uint8_t *out, uint8_t *scores, uint8_t *probs, int row_stride, void *workspace,
                            size_t workspace_bytes, uint8_t *k_levels_out, uint8_t *v_levels_out, uint8_t *amin_out,
                            int bsz, int n_kv_heads, int n_max_blocks, int max_seq_len, int head_dim, int d_block,
                            int top_max_k, int cur_len, int rest_start, int rest_len, int reference,
                            int flags, akv_stream_t stream);

/*
 * akv_decode_step for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as akv_decode_step
 * without `workspace` / `workspace_bytes`: the step's scratch (probe exponents, thresholds, tail outputs, partial sums of
 * the V pass) lives in an array of AKV_STATIC_SCRATCH_BYTES bytes inside the library's device code, one copy per GPU,
 * held until the process ends.  The call allocates and frees nothing.  Shapes for which
 * akv_decode_step_workspace_bytes(bsz, n_kv_heads, head_dim, max_seq_len) exceeds AKV_STATIC_SCRATCH_BYTES are rejected
 * (AKV_ERR_INVALID).  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two streams,
 * two host threads) race on it and must be serialised by the caller; nothing in the array has to survive between calls.
 * The first call on a device looks the array's address up (hipGetSymbolAddress), which may load the library's device
 * code on that device: make that one call outside stream capture; every later call only launches kernels.  The array
 * is part of the device code of the fused step: a GPU on which the library runs any fused step holds these
 * AKV_STATIC_SCRATCH_BYTES whether or not this entry point is ever called.
 */
#define AKV_STATIC_SCRATCH_BYTES ((size_t)32 << 20)
AKV_API int akv_decode_step_static(uint8_t *k_first_8, uint8_t *k_mid_4, uint8_t *k_last_4, uint8_t *v_first_8,
                                   uint8_t *v_mid_4, uint8_t *v_last_4, uint8_t *k_exp_column_max,
                                   uint8_t *v_exp_column_max, uint8_t *restk, uint8_t *restv, const uint8_t *q,
                                   const uint8_t *k_new, const uint8_t *v_new, const uint8_t *mask, int mask_stride,
                                   uint8_t *out, uint8_t *scores, uint8_t *probs, int row_stride,
                                   uint8_t *k_levels_out, uint8_t *v_levels_out, uint8_t *amin_out,
                                   int bsz, int n_kv_heads, int n_max_blocks, int max_seq_len, int head_dim, int d_block,
                                   int top_max_k, int cur_len, int rest_start, int rest_len, int reference,
                                   int flags, akv_stream_t stream);

/*
 * The fused decode step for grouped-query attention and per-sequence lengths; beyond the reference, which
 * asserts multi-head attention and keeps one scalar length per layer (model/KVCache_AlignedKV.py:32,
 * extension/k_cache_file.py:133, extension/v_cache_file.py:146).  Per query head the algorithm is the
 * reference's, on the planes of KV head (query head / group size): q, out [bsz,1,n_q_heads,head_dim];
 * k_new, v_new, planes, column maxima, rest buffers per KV head; scores / probs [bsz, n_q_heads, row_stride];
 * k_levels_out [bsz,n_q_heads,head_dim], v_levels_out [bsz,n_q_heads,(cur_len+1)/64*64], amin_out [bsz,n_q_heads].
 * seq_lens == NULL: every sequence holds cur_len tokens (akv_decode_step is this case with n_q_heads ==
 * n_kv_heads).  seq_lens != NULL: device int32 [bsz], tokens cached per sequence before the step; cur_len is
 * then an upper bound of them (it sizes the launches), a sequence flushes its rest buffer on the step that
 * fills it, and the step increments every entry of seq_lens on the device.
 * k_block: tokens per block of the K planes, [bsz, n_kv_heads, n_max_blocks, head_dim, k_block] (the d_block of
 * akv_k_cache_save / akv_k_cache_compute).  64 is the reference's layout.  256 (head_dim 64 or 128; multi-head, or 2 to
 * 16 query heads per KV head) makes a channel's nibble row a whole 128-byte line, so a skipped row saves exactly its bytes in HBM traffic;
 * tokens still enter the planes 64 at a time (d_block, the length of the rest buffers), as whole tiles inside a block.
 */
AKV_API int akv_decode_step_gqa(uint8_t *k_first_8, uint8_t *k_mid_4, uint8_t *k_last_4, uint8_t *v_first_8,
                                uint8_t *v_mid_4, uint8_t *v_last_4, uint8_t *k_exp_column_max,
                                uint8_t *v_exp_column_max, uint8_t *restk, uint8_t *restv, const uint8_t *q,
                                const uint8_t *k_new, const uint8_t *v_new, const uint8_t *mask, int mask_stride,
                                uint8_t *out, uint8_t *scores, uint8_t *probs, int row_stride, void *workspace,
                                size_t workspace_bytes, uint8_t *k_levels_out, uint8_t *v_levels_out, uint8_t *amin_out,
                                int bsz, int n_q_heads, int n_kv_heads, int n_max_blocks, int max_seq_len, int head_dim,
                                int d_block, int k_block, int top_max_k, int cur_len, int *seq_lens, int reference,
                                int flags, akv_stream_t stream);

/*
 * akv_decode_step_gqa with everything that stays the same from step to step of one layer gathered in a descriptor the
 * caller fills once: a step then passes 15 arguments instead of 38, which is what a host binding pays per call (the
 * reference's Python layer calls its ops once per layer and decode step, model/KVCache_AlignedKV.py:116-124).  Same
 * checks, same kernels, same results as akv_decode_step_gqa with the descriptor's fields in place of its arguments.
 */
typedef struct akv_step_desc {
    uint8_t *k_first_8, *k_mid_4, *k_last_4, *v_first_8, *v_mid_4, *v_last_4;
    uint8_t *k_exp_column_max, *v_exp_column_max, *restk, *restv;
    uint8_t *scores, *probs;
    void *workspace;
    size_t workspace_bytes;
    int row_stride;
    int bsz, n_q_heads, n_kv_heads, n_max_blocks, max_seq_len, head_dim, d_block, k_block, top_max_k;
} akv_step_desc;
AKV_API int akv_decode_step_desc(const akv_step_desc *desc, const uint8_t *q, const uint8_t *k_new, const uint8_t *v_new,
                                 const uint8_t *mask, int mask_stride, uint8_t *out, uint8_t *k_levels_out,
                                 uint8_t *v_levels_out, uint8_t *amin_out, int cur_len, int *seq_lens, int reference,
                                 int flags, akv_stream_t stream);

/*
 * Dense fp16 decode attention, the baseline of the benchmark (semantics of the reference's dense branch,
 * model/Llama_AlignedKV.py:130-139): appends k_new / v_new at row cur_len of the head-major fp16 caches
 * [bsz, heads, max_seq_len, head_dim] and attends over cur_len + 1 tokens.  q, k_new, v_new, out: fp16
 * [bsz,1,heads,head_dim]; scores / probs: fp16 [bsz, heads, row_stride] scratch.  head_dim 128 only.
 */
AKV_API size_t akv_dense_decode_step_workspace_bytes(int bsz, int n_heads, int head_dim, int max_seq_len);
AKV_API int akv_dense_decode_step(uint8_t *k_cache, uint8_t *v_cache, const uint8_t *q, const uint8_t *k_new,
                                  const uint8_t *v_new, uint8_t *out, uint8_t *scores, uint8_t *probs, int row_stride,
                                  void *workspace, size_t workspace_bytes, int bsz, int n_heads, int max_seq_len,
                                  int head_dim, int cur_len, akv_stream_t stream);

/*
 * Benchmark aid, no counterpart in the reference: with profiling enabled, akv_decode_step records HIP
 * events on its stream around its four phases; akv_profile_read waits for the last recorded step and
 * returns the elapsed milliseconds of {K pass, middle, V pass, combine}.  The switch and the events are process-wide
 * and unsynchronised: single-threaded benchmark use only (one host thread, one stream at a time); leave profiling
 * off in a program that runs steps from several threads or streams.
 */
/* The AKV_TUNE_* environment switches are read when first used; call this after changing one in a running process. */
AKV_API int akv_reload_tuning(void);
AKV_API int akv_profile_enable(int enable);
/* Plain device copy of `bytes` bytes (multiple of 16): the known-size kernel hardware byte counters are scaled against. */
AKV_API int akv_copy_probe(void *dst, const void *src, size_t bytes, akv_stream_t stream);
AKV_API int akv_profile_read(float *phase_ms /* [4] */);
/* Interval between two events recorded back to back after the last step: what an event pair measures around
 * nothing.  Subtract it from a phase of akv_profile_read to get the kernel's own duration. */
AKV_API int akv_profile_read_empty(float *empty_ms /* [1] */);

#ifdef __cplusplus
}
#endif
#endif /* ALIGNEDKV_H */
