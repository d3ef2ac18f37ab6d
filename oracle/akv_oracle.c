/*
 * CPU restatement (plain C) of the five AlignedKV extension ops.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT THE PRODUCT: it is the checker for the HIP library and the
 * "port" CPU baseline of the benchmark; nothing in the product path links or loads it.
 *
 * Each function walks the same (grid, thread, loop) index space as the reference kernel it
 * restates and uses the same flat-index expressions, so that a transposed stride or a swapped
 * nibble in the vectorised NumPy restatement shows up as a mismatch against this file.
 * Differences from the reference, on purpose:
 *   - dot products accumulate in fp32 (the reference chains __hfma2 in fp16); the exact fp16
 *     bits of the reference's sums are "parity unpinned" (nothing in the reference pins them);
 *   - the `trick` bytes {0x00, 0x88} are immediates (the reference reads them from shared memory
 *     without a barrier, extension/csrc/K_cache.cu:201-205).
 * Paths cited below are relative to the reference checkout.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define AKVO_API __attribute__((visibility("default")))

/* ---- fp16 <-> fp32, bit exact, round-to-nearest-even ------------------------------------ */
static float half_lut[65536];
static int half_lut_ready = 0;

static float half_bits_to_float_slow(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t out;
    if (exp == 0) {
        if (man == 0) {
            out = sign;
        } else {
            int e = -1;
            do { man <<= 1; ++e; } while ((man & 0x400u) == 0);
            out = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        out = sign | 0x7F800000u | (man << 13);
    } else {
        out = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &out, 4);
    return f;
}

AKVO_API void akvo_init(void) {
    if (half_lut_ready) return;
    for (uint32_t i = 0; i < 65536u; ++i) half_lut[i] = half_bits_to_float_slow((uint16_t)i);
    half_lut_ready = 1;
}

static inline float h2f(uint16_t h) { return half_lut[h]; }

AKVO_API uint16_t akvo_float_to_half(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) {                       /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | ((absx > 0x7F800000u) ? (0x200u | ((absx >> 13) & 0x3FFu)) : 0u));
    }
    if (absx >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);   /* rounds to inf (>= 65520) */
    if (absx < 0x33000001u) return (uint16_t)sign;                /* <= 2^-25 rounds to zero */
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t m = (absx & 0x7FFFFFu) | 0x800000u;
    uint32_t shift, half_exp;
    if (e < -14) { shift = (uint32_t)(13 + (-14 - e)); half_exp = 0; }
    else { shift = 13; half_exp = (uint32_t)(e + 15); }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) ++q;
    uint32_t out = (half_exp == 0) ? q : ((half_exp << 10) + (q - 0x400u));
    return (uint16_t)(sign | out);
}

AKVO_API float akvo_half_to_float(uint16_t h) { return half_bits_to_float_slow(h); }

/* ---- k_cache_save : extension/csrc/K_cache.cu:19-58 (prefill), :63-94 (decoding), :97-164 --- */
AKVO_API void akvo_k_cache_save(uint8_t *first_8, uint8_t *mid_4, uint8_t *last_4, const uint8_t *k_new,
                                int bsz, int n_kv_heads, int n_blocks, int n_max_blocks, int d_head,
                                int d_block, int start_pos, int seqlen) {
    const int64_t stride_dim = d_block >> 1;                       /* K_cache.cu:113-119 */
    const int64_t stride_block = stride_dim * d_head;
    const int64_t stride_head = stride_block * n_max_blocks;
    const int64_t stride_batch = stride_head * n_kv_heads;
    const int64_t nstride_head = d_head;
    const int64_t nstride_seq = nstride_head * n_kv_heads;
    const int64_t nstride_batch = nstride_seq * seqlen;
    if (start_pos == 0 || seqlen % d_block == 0) {
        if (n_blocks == 0) return;
        const int start_pos_block = start_pos / d_block;
        for (int bx = 0; bx < bsz; ++bx)
        for (int by = 0; by < n_kv_heads; ++by)
        for (int bz = 0; bz < n_blocks; ++bz)
        for (int tx = 0; tx < d_head; ++tx) {
            int block_start_seq = bz * d_block;
            int block_end_seq = block_start_seq + d_block < seqlen ? block_start_seq + d_block : seqlen;
            for (int seq = block_start_seq; seq < block_end_seq; ++seq) {
                int first_8_index = seq - block_start_seq;
                int mid_4_index = first_8_index >> 1;
                int move = (first_8_index & 1) << 2;
                int64_t base = bx * stride_batch + by * stride_head + (int64_t)(bz + start_pos_block) * stride_block + tx * stride_dim;
                int64_t src = (bx * nstride_batch + seq * nstride_seq + by * nstride_head + tx) * 2;
                first_8[base * 2 + first_8_index] = k_new[src + 1];
                mid_4[base + mid_4_index] += (uint8_t)((k_new[src] & 0xf0) >> move);
                last_4[base + mid_4_index] += (uint8_t)((k_new[src] & 0x0f) << (4 - move));
            }
        }
    } else if (seqlen == 1) {
        const int block_pos = start_pos / d_block;
        const int first_8_index = start_pos - block_pos * d_block;
        const int mid_4_index = first_8_index >> 1;
        const int move = (first_8_index & 1) << 2;
        for (int bx = 0; bx < bsz; ++bx)
        for (int by = 0; by < n_kv_heads; ++by)
        for (int tx = 0; tx < d_head; ++tx) {
            int64_t base = bx * stride_batch + by * stride_head + (int64_t)block_pos * stride_block + tx * stride_dim;
            int64_t src = (bx * nstride_batch + by * nstride_head + tx) * 2;
            first_8[base * 2 + first_8_index] = k_new[src + 1];
            mid_4[base + mid_4_index] += (uint8_t)((k_new[src] & 0xf0) >> move);
            last_4[base + mid_4_index] += (uint8_t)((k_new[src] & 0x0f) << (4 - move));
        }
    }
}

/* ---- k_cache_compute : extension/csrc/K_cache.cu:174-310, :314-395 ---------------------------
 * s is written as fp16 bits; row stride of s is (n_blocks+1)*d_block halves.
 * levels_out (may be NULL): uint8 [bsz, n_kv_heads, d_head], the fetch level used per channel. */
AKVO_API void akvo_k_cache_compute(const uint8_t *first_8, const uint8_t *mid_4, const uint8_t *last_4,
                                   const uint8_t *sum_u8, const uint8_t *max_u8, const uint16_t *q,
                                   uint16_t *s, uint8_t *levels_out, int bsz, int n_kv_heads, int n_blocks,
                                   int n_max_blocks, int d_head, int d_block, float sqrt_dim, int reference) {
    akvo_init();
    if (n_blocks == 0) return;
    const int64_t stride_dim = d_block >> 1;                       /* K_cache.cu:341-349 */
    const int64_t stride_block = stride_dim * d_head;
    const int64_t stride_head = stride_block * n_max_blocks;
    const int64_t stride_batch = stride_head * n_kv_heads;
    const int64_t stride_head_q = d_head;
    const int64_t stride_batch_q = stride_head_q * n_kv_heads;
    const int64_t stride_head_s = (int64_t)(n_blocks + 1) * d_block;
    const int64_t stride_batch_s = stride_head_s * n_kv_heads;
    const float scale = h2f(akvo_float_to_half(sqrt_dim));         /* __float2half2_rn(sqrt_dim), :306 */
    const uint8_t trick[2] = {0x00, 0x88};
#pragma omp parallel for collapse(2) schedule(static)
    for (int bx = 0; bx < bsz; ++bx)
    for (int head = 0; head < n_kv_heads; ++head) {               /* blockIdx.y*4 + threadIdx.y */
        const uint8_t mx = max_u8[bx * n_kv_heads + head];
        for (int bz = 0; bz < n_blocks; ++bz)
        for (int tx = 0; tx < (d_block >> 1); ++tx) {
            const int first_8_index_1 = tx << 1, first_8_index_2 = first_8_index_1 + 1, mid_4_index = tx;
            float r1 = 0.f, r2 = 0.f;
            for (int i = 0; i < d_head; ++i) {
                int64_t base = bx * stride_batch + head * stride_head + bz * stride_block + i * stride_dim;
                uint8_t diff = reference ? 0 : (uint8_t)(mx - sum_u8[bx * stride_batch_q + head * stride_head_q + i]);
                const uint8_t *p1 = &first_8[base * 2 + first_8_index_1];
                const uint8_t *p2 = &first_8[base * 2 + first_8_index_2];
                const uint8_t *pm = diff >= 8 ? &trick[1] : &mid_4[base + mid_4_index];
                const uint8_t *pl = diff >= 4 ? (diff >= 8 ? &trick[0] : &trick[1]) : &last_4[base + mid_4_index];
                uint16_t k1 = (uint16_t)((((uint16_t)*p1) << 8) + (((uint16_t)*pm) & 0xf0) + ((((uint16_t)*pl) & 0xf0) >> 4));
                uint16_t k2 = (uint16_t)((((uint16_t)*p2) << 8) + ((((uint16_t)*pm) & 0x0f) << 4) + (((uint16_t)*pl) & 0x0f));
                float qf = h2f(q[bx * stride_batch_q + head * stride_head_q + i]);
                r1 = fmaf(h2f(k1), qf, r1);
                r2 = fmaf(h2f(k2), qf, r2);
                if (levels_out && bz == 0 && tx == 0)
                    levels_out[(bx * n_kv_heads + head) * d_head + i] = diff >= 8 ? 2 : (diff >= 4 ? 1 : 0);
            }
            int seq = bz * d_block + tx * 2;
            s[bx * stride_batch_s + head * stride_head_s + seq] = akvo_float_to_half(r1 * scale);
            s[bx * stride_batch_s + head * stride_head_s + seq + 1] = akvo_float_to_half(r2 * scale);
        }
    }
}

/* ---- v_cache_save : extension/csrc/V_cache.cu:17-41, :44-80 ---------------------------------
 * v_new_seq is v_new.size(1) (the token stride of the source), seq_len the number stored. */
AKVO_API void akvo_v_cache_save(uint8_t *first_8, uint8_t *mid_4, uint8_t *last_4, const uint8_t *v_new,
                                int bsz, int n_heads, int max_seq_len, int head_dim, int start_pos,
                                int seq_len, int v_new_seq) {
    if (seq_len == 0) return;
    const int64_t stride_seq = head_dim >> 1;
    const int64_t stride_head = stride_seq * max_seq_len;
    const int64_t stride_batch = stride_head * n_heads;
    const int64_t nstride_head = head_dim;
    const int64_t nstride_seq = nstride_head * n_heads;
    const int64_t nstride_batch = nstride_seq * v_new_seq;
    for (int bx = 0; bx < bsz; ++bx)
    for (int by = 0; by < n_heads; ++by)
    for (int tx = 0; tx < (head_dim >> 1); ++tx)
    for (int pos = 0; pos < seq_len; ++pos) {
        int64_t dst = bx * stride_batch + by * stride_head + (int64_t)(pos + start_pos) * stride_seq + tx;
        int64_t src0 = (bx * nstride_batch + pos * nstride_seq + by * nstride_head + tx * 2) * 2;
        int64_t src1 = (bx * nstride_batch + pos * nstride_seq + by * nstride_head + tx * 2 + 1) * 2;
        first_8[dst * 2] = v_new[src0 + 1];
        first_8[dst * 2 + 1] = v_new[src1 + 1];
        mid_4[dst] = (uint8_t)((v_new[src0] & 0xf0) + ((v_new[src1] & 0xf0) >> 4));
        last_4[dst] = (uint8_t)(((v_new[src0] & 0x0f) << 4) + (v_new[src1] & 0x0f));
    }
}

/* ---- v_cache_test_compute : extension/csrc/V_cache.cu:90-123, :125-168 ---------------------- */
AKVO_API void akvo_v_cache_test_compute(const uint8_t *first_8, const uint16_t *test_s_value,
                                        const int32_t *test_s_index, uint16_t *test_o, int bsz, int n_heads,
                                        int max_seq_len, int head_dim, int top_max_k) {
    akvo_init();
    const int64_t stride_seq = head_dim >> 1;
    const int64_t stride_head = stride_seq * max_seq_len;
    const int64_t stride_batch = stride_head * n_heads;
    for (int bx = 0; bx < bsz; ++bx)
    for (int by = 0; by < n_heads; ++by)
    for (int tx = 0; tx < (head_dim >> 1); ++tx) {
        float r1 = 0.f, r2 = 0.f;
        for (int i = 0; i < top_max_k; ++i) {
            uint16_t v1 = 0x0080, v2 = 0x0080;
            int64_t index = (int64_t)test_s_index[(bx * n_heads + by) * top_max_k + i] * top_max_k + i;
            int64_t at = (bx * stride_batch + by * stride_head + index * stride_seq + tx) * 2;
            v1 = (uint16_t)(v1 + (((uint16_t)first_8[at]) << 8));
            v2 = (uint16_t)(v2 + (((uint16_t)first_8[at + 1]) << 8));
            v1 &= 0x7FFF;
            v2 &= 0x7FFF;
            float sf = h2f(test_s_value[(bx * n_heads + by) * top_max_k + i]);
            r1 = fmaf(h2f(v1), sf, r1);
            r2 = fmaf(h2f(v2), sf, r2);
        }
        test_o[(bx * n_heads + by) * head_dim + tx * 2] = akvo_float_to_half(r1);
        test_o[(bx * n_heads + by) * head_dim + tx * 2 + 1] = akvo_float_to_half(r2);
    }
}

/* ---- v_cache_compute : extension/csrc/V_cache.cu:178-308, :310-374 --------------------------
 * s_last_dim is the row stride of s in halves; levels_out (may be NULL): uint8 [bsz,n_heads,n_tokens]. */
AKVO_API void akvo_v_cache_compute(const uint8_t *first_8, const uint8_t *mid_4, const uint8_t *last_4,
                                   const uint16_t *s, const uint8_t *amin_u8, uint16_t *o, uint8_t *levels_out,
                                   int bsz, int n_heads, int max_seq_len, int head_dim, int s_last_dim,
                                   int n_tokens, int reference) {
    akvo_init();
    const int64_t stride_seq = head_dim >> 1;
    const int64_t stride_head = stride_seq * max_seq_len;
    const int64_t stride_batch = stride_head * n_heads;
    const int64_t stride_head_s = s_last_dim;
    const int64_t stride_batch_s = stride_head_s * n_heads;
    const uint8_t trick[2] = {0x00, 0x88};
#pragma omp parallel for collapse(2) schedule(static)
    for (int bx = 0; bx < bsz; ++bx)
    for (int by = 0; by < n_heads; ++by) {
        short amin = (short)amin_u8[bx * n_heads + by];           /* V_cache.cu:195-197 */
        amin = (short)(amin << 10);
        for (int tx = 0; tx < (head_dim >> 1); ++tx) {
            float r1 = 0.f, r2 = 0.f;
            for (int i = 0; i < n_tokens; ++i) {
                uint16_t sb = s[bx * stride_batch_s + by * stride_head_s + i];
                short diff = reference ? (short)0 : (short)(amin - (short)sb);   /* :211 */
                int64_t at = bx * stride_batch + by * stride_head + (int64_t)i * stride_seq + tx;
                const uint8_t *p1 = &first_8[at * 2];
                const uint8_t *p2 = &first_8[at * 2 + 1];
                const uint8_t *pm = diff >= 0x0800 ? &trick[1] : &mid_4[at];
                const uint8_t *pl = diff >= 0x0400 ? (diff >= 0x0800 ? &trick[0] : &trick[1]) : &last_4[at];
                uint16_t v1 = (uint16_t)((((uint16_t)*p1) << 8) + (((uint16_t)*pm) & 0xf0) + ((((uint16_t)*pl) & 0xf0) >> 4));
                uint16_t v2 = (uint16_t)((((uint16_t)*p2) << 8) + ((((uint16_t)*pm) & 0x0f) << 4) + (((uint16_t)*pl) & 0x0f));
                float sf = h2f(sb);
                r1 = fmaf(h2f(v1), sf, r1);
                r2 = fmaf(h2f(v2), sf, r2);
                if (levels_out && tx == 0)
                    levels_out[((int64_t)bx * n_heads + by) * n_tokens + i] = diff >= 0x0800 ? 2 : (diff >= 0x0400 ? 1 : 0);
            }
            o[(bx * n_heads + by) * head_dim + tx * 2] = akvo_float_to_half(r1);
            o[(bx * n_heads + by) * head_dim + tx * 2 + 1] = akvo_float_to_half(r2);
        }
    }
}

/* ---- dense fp16 decode attention, the semantics of model/Llama_AlignedKV.py:130-139 ----------
 * q [B,H,D], k/v [B,L,H,D] fp16 bits, out [B,H,D]; fp32 accumulate, fp16 roundings where the
 * PyTorch expression materialises fp16 tensors. */
AKVO_API void akvo_dense_attention(const uint16_t *q, const uint16_t *k, const uint16_t *v, uint16_t *out,
                                   float *scratch, int bsz, int n_heads, int seq, int head_dim) {
    akvo_init();
    const float inv = sqrtf((float)head_dim);
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < bsz; ++b)
    for (int h = 0; h < n_heads; ++h) {
        float *w = scratch + ((int64_t)b * n_heads + h) * seq;
        const uint16_t *qq = q + ((int64_t)b * n_heads + h) * head_dim;
        float mx = -INFINITY;
        for (int t = 0; t < seq; ++t) {
            const uint16_t *kk = k + (((int64_t)b * seq + t) * n_heads + h) * head_dim;
            float acc = 0.f;
            for (int d = 0; d < head_dim; ++d) acc = fmaf(h2f(kk[d]), h2f(qq[d]), acc);
            float sc = h2f(akvo_float_to_half(h2f(akvo_float_to_half(acc)) / inv));
            w[t] = sc;
            mx = sc > mx ? sc : mx;
        }
        float sum = 0.f;
        for (int t = 0; t < seq; ++t) { w[t] = expf(w[t] - mx); sum += w[t]; }
        for (int t = 0; t < seq; ++t) w[t] = h2f(akvo_float_to_half(w[t] / sum));
        for (int d = 0; d < head_dim; ++d) {
            float acc = 0.f;
            for (int t = 0; t < seq; ++t)
                acc = fmaf(h2f(v[(((int64_t)b * seq + t) * n_heads + h) * head_dim + d]), w[t], acc);
            out[((int64_t)b * n_heads + h) * head_dim + d] = akvo_float_to_half(acc);
        }
    }
}

AKVO_API int akvo_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
