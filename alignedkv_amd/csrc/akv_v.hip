// V side of the AlignedKV hot path: plane writes (v_cache_save), the output-magnitude probe
// (v_cache_test_compute) and the decode output GEMV (v_cache_compute).
//
// Plane layout (reference: extension/v_cache_file.py:46-54): token-major rows, first_8[t][d]
// (head_dim bytes per token) and mid_4/last_4[t][d/2] (even channel in the high nibble).
//
// Output kernel, tuned shape (head_dim in {64,128,256}): the sequence is split into chunks, one
// workgroup of 4 waves per (batch, head, chunk).  A 16-byte load per lane covers 64/(D/16) token
// rows of first_8 (lane = 16 channels of one token), an 8-byte load covers the same channels of
// a nibble row.  The fetch level depends only on the token, i.e. on lane/(D/16): nibble loads of
// skipped tokens get an out-of-range buffer offset (return 0, fetch nothing) and are OR-ed with
// the substitution byte.  Each lane keeps 16 fp32 accumulators (its channels); a reduce-scatter
// over the lanes that share channels, LDS across the 4 waves, then fp32 partial sums per chunk
// that a second small kernel adds up in a fixed order (deterministic output bits).
#include "akv_cores.h"

namespace akv {

// ------------------------------------------------------------------------------------------------
// v_cache_save.  reference: extension/csrc/V_cache.cu:17-41.
// one thread per 8 channels of one token (16 bytes in, 8 + 4 + 4 bytes out)
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void v_save_vec8_kernel(uint8_t *__restrict__ first_8, uint8_t *__restrict__ mid_4,
                                                          uint8_t *__restrict__ last_4,
                                                          const unsigned short *__restrict__ v_new, int H, int D,
                                                          int max_seq_len, int start_pos, int seq_len, int v_new_seq,
                                                          int64_t total) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int d8n = D >> 3;
    int d8 = (int)(idx % d8n);
    int64_t r = idx / d8n;
    int h = (int)(r % H);
    r /= H;
    int pos = (int)(r % seq_len);
    int b = (int)(r / seq_len);
    u32x4 w = *reinterpret_cast<const u32x4 *>(v_new + (((int64_t)b * v_new_seq + pos) * H + h) * D + d8 * 8);
    // w.x = channels (0,1), w.y = (2,3), ...; each half = lo byte | hi byte << 8
    u32 ww[4] = {w.x, w.y, w.z, w.w};
    u32 hi0 = 0, hi1 = 0, mid = 0, last = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        u32 e = ww[i] & 0xffffu, o = ww[i] >> 16;   // even / odd channel of the pair
        u32 hpair = (e >> 8) | ((o >> 8) << 8);
        if (i < 2) hi0 |= hpair << (16 * i); else hi1 |= hpair << (16 * (i - 2));
        mid |= ((e & 0xf0u) | ((o & 0xf0u) >> 4)) << (8 * i);
        last |= (((e & 0x0fu) << 4) | (o & 0x0fu)) << (8 * i);
    }
    int64_t row = ((int64_t)b * H + h) * max_seq_len + start_pos + pos;
    u32x2 hv = {hi0, hi1};
    *reinterpret_cast<u32x2 *>(first_8 + row * D + d8 * 8) = hv;
    *reinterpret_cast<u32 *>(mid_4 + row * (D >> 1) + d8 * 4) = mid;
    *reinterpret_cast<u32 *>(last_4 + row * (D >> 1) + d8 * 4) = last;
}

// any even head_dim: one thread per channel pair
__global__ __launch_bounds__(256) void v_save_pair_kernel(uint8_t *__restrict__ first_8, uint8_t *__restrict__ mid_4,
                                                          uint8_t *__restrict__ last_4,
                                                          const unsigned short *__restrict__ v_new, int H, int D,
                                                          int max_seq_len, int start_pos, int seq_len, int v_new_seq,
                                                          int64_t total) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int d2n = D >> 1;
    int d2 = (int)(idx % d2n);
    int64_t r = idx / d2n;
    int h = (int)(r % H);
    r /= H;
    int pos = (int)(r % seq_len);
    int b = (int)(r / seq_len);
    const unsigned short *src = v_new + (((int64_t)b * v_new_seq + pos) * H + h) * D + d2 * 2;
    u32 e = src[0], o = src[1];
    int64_t row = ((int64_t)b * H + h) * max_seq_len + start_pos + pos;
    first_8[row * D + d2 * 2] = (uint8_t)(e >> 8);
    first_8[row * D + d2 * 2 + 1] = (uint8_t)(o >> 8);
    mid_4[row * d2n + d2] = (uint8_t)((e & 0xf0u) | ((o & 0xf0u) >> 4));
    last_4[row * d2n + d2] = (uint8_t)(((e & 0x0fu) << 4) | (o & 0x0fu));
}

// ------------------------------------------------------------------------------------------------
// v_cache_test_compute.  reference: extension/csrc/V_cache.cu:90-123.  grid (H, B), one thread per
// channel; token indices are clamped into the plane.
// ------------------------------------------------------------------------------------------------
__global__ void v_test_kernel(const uint8_t *__restrict__ first_8, const unsigned short *__restrict__ s_val,
                              const int *__restrict__ s_idx, unsigned short *__restrict__ test_o, int H, int D,
                              int max_seq_len, int top_k) {
    const int h = blockIdx.x, b = blockIdx.y;
    const int bh = b * H + h;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        float acc = 0.f;
        for (int i = 0; i < top_k; ++i) {
            int64_t tok = (int64_t)s_idx[(int64_t)bh * top_k + i] * top_k + i;
            tok = tok < 0 ? 0 : (tok >= max_seq_len ? max_seq_len - 1 : tok);
            u32 hi = first_8[((int64_t)bh * max_seq_len + tok) * D + d];
            u32 bits = ((hi << 8) | 0x80u) & 0x7fffu;
            acc = fmaf(half_bits_to_float(bits), half_bits_to_float(s_val[(int64_t)bh * top_k + i]), acc);
        }
        test_o[(int64_t)bh * D + d] = float_to_half_bits(acc);
    }
}

// ------------------------------------------------------------------------------------------------
// v_cache_compute
// ------------------------------------------------------------------------------------------------
// grid (n_chunks, H, B), 256 threads.  partial: fp32 [B*H, n_chunks, D].
template <int D, bool REF, int NIT>
__global__ __launch_bounds__(256) void v_compute_tuned_kernel(
    const uint8_t *__restrict__ first_8, const uint8_t *__restrict__ mid_4, const uint8_t *__restrict__ last_4,
    const unsigned short *__restrict__ s, const uint8_t *__restrict__ amin_u8, float *__restrict__ partial,
    uint8_t *__restrict__ levels_out, int H, int max_seq_len, int s_last_dim, int n_tokens, int tokens_per_wave,
    int n_chunks) {
    __shared__ float wave_part[4][D];
    const int wave = wave_index();
    const int chunk = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int bh = b * H + h;
    const int t_begin = (chunk * 4 + wave) * tokens_per_wave;
    const int t_end = min(t_begin + tokens_per_wave, n_tokens);
    const int64_t row0 = (int64_t)bh * max_seq_len;
    VFirstTile<D> ft;
    v_prefetch_first<D>(ft, first_8 + row0 * D, n_tokens, t_begin, t_end);
    const unsigned char amin = REF ? 0 : amin_u8[bh];
    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    v_accumulate<D, REF, NIT>(ft, first_8 + row0 * D, mid_4 + row0 * (D / 2), last_4 + row0 * (D / 2), n_tokens,
                         s + (int64_t)bh * s_last_dim, amin, t_begin, t_end, acc,
                         levels_out != nullptr ? levels_out + (int64_t)bh * n_tokens : nullptr);
    v_fold_workgroup<D>(acc, wave_part, partial + ((int64_t)bh * n_chunks + chunk) * D);
}

// any even head_dim: grid (n_chunks, H, B), one thread per channel pair, serial over the chunk's tokens.
template <bool REF>
__global__ void v_compute_generic_kernel(const uint8_t *__restrict__ first_8, const uint8_t *__restrict__ mid_4,
                                         const uint8_t *__restrict__ last_4, const unsigned short *__restrict__ s,
                                         const uint8_t *__restrict__ amin_u8, float *__restrict__ partial,
                                         uint8_t *__restrict__ levels_out, int H, int D, int max_seq_len,
                                         int s_last_dim, int n_tokens, int chunk_tokens, int n_chunks) {
    const int chunk = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int bh = b * H + h;
    const unsigned char amin = REF ? 0 : amin_u8[bh];
    const int t0 = chunk * chunk_tokens, t1 = min(t0 + chunk_tokens, n_tokens);
    for (int tx = threadIdx.x; tx < (D >> 1); tx += blockDim.x) {
        float r1 = 0.f, r2 = 0.f;
        for (int t = t0; t < t1; ++t) {
            u32 sbits = s[(int64_t)bh * s_last_dim + t];
            int lv = REF ? 0 : v_level(amin, (unsigned short)sbits);
            if (levels_out != nullptr && tx == 0) levels_out[(int64_t)bh * n_tokens + t] = (uint8_t)lv;
            int64_t row = (int64_t)bh * max_seq_len + t;
            u32 h1 = first_8[row * D + 2 * tx], h2 = first_8[row * D + 2 * tx + 1];
            u32 m = lv < 2 ? mid_4[row * (D >> 1) + tx] : 0u;
            u32 l = lv == 0 ? last_4[row * (D >> 1) + tx] : 0u;
            float sf = half_bits_to_float(sbits);
            r1 = fmaf(half_bits_to_float(rebuild_bits(h1, m >> 4, l >> 4, lv)), sf, r1);
            r2 = fmaf(half_bits_to_float(rebuild_bits(h2, m & 0xfu, l & 0xfu, lv)), sf, r2);
        }
        partial[((int64_t)bh * n_chunks + chunk) * D + 2 * tx] = r1;
        partial[((int64_t)bh * n_chunks + chunk) * D + 2 * tx + 1] = r2;
    }
}

// grid (B*H), D threads (strided): o = fp16(sum of the chunk partials in chunk order).
__global__ void v_combine_kernel(const float *__restrict__ partial, unsigned short *__restrict__ o, int D, int n_chunks) {
    const int bh = blockIdx.x;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        float acc = 0.f;
        for (int c = 0; c < n_chunks; ++c) acc += partial[((int64_t)bh * n_chunks + c) * D + d];
        o[(int64_t)bh * D + d] = float_to_half_bits(acc);
    }
}

template <int D, bool REF, int NIT>
static void launch_v_tuned_nit(const uint8_t *f8, const uint8_t *m4, const uint8_t *l4, const uint8_t *s,
                               const uint8_t *amin, float *partial, uint8_t *levels, int B, int H, int max_seq_len,
                               int s_last_dim, int n_tokens, const VPlan &p, hipStream_t st) {
    hipLaunchKernelGGL((v_compute_tuned_kernel<D, REF, NIT>), dim3(p.n_chunks, H, B), dim3(256), 0, st, f8, m4, l4,
                       reinterpret_cast<const unsigned short *>(s), amin, partial, levels, H, max_seq_len, s_last_dim,
                       n_tokens, p.tokens_per_wave, p.n_chunks);
}

template <int D>
static void launch_v_tuned(bool ref, const uint8_t *f8, const uint8_t *m4, const uint8_t *l4, const uint8_t *s,
                           const uint8_t *amin, float *partial, uint8_t *levels, int B, int H, int max_seq_len,
                           int s_last_dim, int n_tokens, const VPlan &p, hipStream_t st) {
#define AKV_V_CASE(R, N)                                                                                       \
    launch_v_tuned_nit<D, R, N>(f8, m4, l4, s, amin, partial, levels, B, H, max_seq_len, s_last_dim, n_tokens, p, st)
    if (ref) {
        if (p.iters_per_wave == 1) AKV_V_CASE(true, 1);
        else if (p.iters_per_wave == 2) AKV_V_CASE(true, 2);
        else AKV_V_CASE(true, 4);
    } else {
        if (p.iters_per_wave == 1) AKV_V_CASE(false, 1);
        else if (p.iters_per_wave == 2) AKV_V_CASE(false, 2);
        else AKV_V_CASE(false, 4);
    }
#undef AKV_V_CASE
}

}  // namespace akv

using namespace akv;

namespace akv {
int launch_v_save(uint8_t *first_8, uint8_t *mid_4, uint8_t *last_4, const uint8_t *v_new, int bsz, int n_local_kv_heads,
                  int max_seq_len, int head_dim, int start_pos, int seq_len, int v_new_seq, hipStream_t st) {
    if (seq_len == 0) return AKV_OK;   // reference: extension/csrc/V_cache.cu:54-55
    AKV_REQUIRE(first_8 && mid_4 && last_4 && v_new, "v_cache_save: null pointer");
    AKV_REQUIRE(bsz > 0 && n_local_kv_heads > 0 && max_seq_len > 0 && head_dim > 0 && head_dim % 2 == 0,
                "v_cache_save: bad dimension (bsz=%d heads=%d max_seq_len=%d head_dim=%d)", bsz, n_local_kv_heads,
                max_seq_len, head_dim);
    AKV_REQUIRE(seq_len > 0 && start_pos >= 0 && start_pos + seq_len <= max_seq_len,
                "v_cache_save: rows %d..%d outside the plane of %d rows", start_pos, start_pos + seq_len, max_seq_len);
    AKV_REQUIRE(v_new_seq >= seq_len, "v_cache_save: v_new holds %d tokens, %d requested", v_new_seq, seq_len);
    const unsigned short *src = reinterpret_cast<const unsigned short *>(v_new);
    if (head_dim % 8 == 0) {
        int64_t total = (int64_t)bsz * seq_len * n_local_kv_heads * (head_dim / 8);
        hipLaunchKernelGGL(v_save_vec8_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, first_8, mid_4,
                           last_4, src, n_local_kv_heads, head_dim, max_seq_len, start_pos, seq_len, v_new_seq, total);
    } else {
        int64_t total = (int64_t)bsz * seq_len * n_local_kv_heads * (head_dim / 2);
        hipLaunchKernelGGL(v_save_pair_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, first_8, mid_4,
                           last_4, src, n_local_kv_heads, head_dim, max_seq_len, start_pos, seq_len, v_new_seq, total);
    }
    return check_launch("v_cache_save");
}
}  // namespace akv

extern "C" int akv_v_cache_save(uint8_t *first_8, uint8_t *mid_4, uint8_t *last_4, const uint8_t *v_new, int bsz,
                                int n_local_kv_heads, int max_seq_len, int head_dim, int start_pos, int seq_len,
                                int v_new_seq, akv_stream_t stream) {
    return launch_v_save(first_8, mid_4, last_4, v_new, bsz, n_local_kv_heads, max_seq_len, head_dim, start_pos, seq_len,
                         v_new_seq, static_cast<hipStream_t>(stream));
}

extern "C" int akv_v_cache_test_compute(const uint8_t *first_8, const uint8_t *mid_4, const uint8_t *last_4,
                                        const uint8_t *test_s_value, const uint8_t *test_s_index,
                                        uint8_t *test_o_out, int bsz, int n_local_kv_heads, int max_seq_len,
                                        int head_dim, int top_max_k, akv_stream_t stream) {
    (void)mid_4;
    (void)last_4;   // the probe reads the high-byte plane only (extension/csrc/V_cache.cu:108-112)
    AKV_REQUIRE(first_8 && test_s_value && test_s_index && test_o_out, "v_cache_test_compute: null pointer");
    AKV_REQUIRE(bsz > 0 && n_local_kv_heads > 0 && max_seq_len > 0 && head_dim > 0 && top_max_k > 0,
                "v_cache_test_compute: bad dimension");
    AKV_REQUIRE(bsz <= 65535, "v_cache_test_compute: bsz exceeds the grid limit 65535");
    hipLaunchKernelGGL(v_test_kernel, dim3(n_local_kv_heads, bsz), dim3(head_dim < 256 ? head_dim : 256), 0,
                       static_cast<hipStream_t>(stream), first_8, reinterpret_cast<const unsigned short *>(test_s_value),
                       reinterpret_cast<const int *>(test_s_index), reinterpret_cast<unsigned short *>(test_o_out),
                       n_local_kv_heads, head_dim, max_seq_len, top_max_k);
    return check_launch("v_cache_test_compute");
}

extern "C" size_t akv_v_cache_compute_workspace_bytes(int bsz, int n_local_kv_heads, int head_dim, int n_tokens) {
    if (bsz <= 0 || n_local_kv_heads <= 0 || head_dim <= 0 || n_tokens < 0) return 0;
    VPlan p = v_plan(bsz, n_local_kv_heads, head_dim, n_tokens);
    size_t n = (size_t)bsz * n_local_kv_heads * (size_t)(p.n_chunks > 0 ? p.n_chunks : 1) * head_dim * sizeof(float);
    return (n + 255) & ~(size_t)255;
}

extern "C" int akv_v_cache_compute(const uint8_t *first_8, const uint8_t *mid_4, const uint8_t *last_4,
                                   const uint8_t *s, const uint8_t *amin, uint8_t *o_out, uint8_t *levels_out,
                                   void *workspace, size_t workspace_bytes, int bsz, int n_local_kv_heads,
                                   int max_seq_len, int head_dim, int s_last_dim, int start_pos_add_seqlen,
                                   int reference, akv_stream_t stream) {
    const int n_tokens = start_pos_add_seqlen;
    AKV_REQUIRE(first_8 && mid_4 && last_4 && o_out, "v_cache_compute: null pointer");
    AKV_REQUIRE(bsz > 0 && n_local_kv_heads > 0 && max_seq_len > 0 && head_dim > 0 && head_dim % 2 == 0,
                "v_cache_compute: bad dimension (bsz=%d heads=%d max_seq_len=%d head_dim=%d)", bsz, n_local_kv_heads,
                max_seq_len, head_dim);
    AKV_REQUIRE(n_tokens >= 0 && n_tokens <= max_seq_len, "v_cache_compute: %d tokens requested, plane holds %d",
                n_tokens, max_seq_len);
    AKV_REQUIRE(n_tokens == 0 || (s != nullptr && s_last_dim >= n_tokens),
                "v_cache_compute: s row stride %d shorter than %d tokens", s_last_dim, n_tokens);
    AKV_REQUIRE(reference || n_tokens == 0 || amin != nullptr, "v_cache_compute: null alignment pointer");
    AKV_REQUIRE(bsz <= 65535 && n_local_kv_heads <= 65535, "v_cache_compute: bsz/heads exceed the grid limit 65535");
    AKV_REQUIRE((int64_t)max_seq_len * head_dim < (int64_t)1 << 31,
                "v_cache_compute: one (batch, head) slice of first_8 must stay below 2 GiB");
    const size_t need = akv_v_cache_compute_workspace_bytes(bsz, n_local_kv_heads, head_dim, n_tokens);
    AKV_REQUIRE(workspace != nullptr && workspace_bytes >= need, "v_cache_compute: workspace of %zu bytes, %zu needed",
                workspace_bytes, need);
    hipStream_t st = static_cast<hipStream_t>(stream);
    VPlan p = v_plan(bsz, n_local_kv_heads, head_dim, n_tokens);
    float *partial = static_cast<float *>(workspace);
    const bool ref = reference != 0;
    if (p.n_chunks > 0) {
        if (p.tuned) {
            if (head_dim == 64)
                launch_v_tuned<64>(ref, first_8, mid_4, last_4, s, amin, partial, levels_out, bsz, n_local_kv_heads,
                                   max_seq_len, s_last_dim, n_tokens, p, st);
            else if (head_dim == 128)
                launch_v_tuned<128>(ref, first_8, mid_4, last_4, s, amin, partial, levels_out, bsz, n_local_kv_heads,
                                    max_seq_len, s_last_dim, n_tokens, p, st);
            else
                launch_v_tuned<256>(ref, first_8, mid_4, last_4, s, amin, partial, levels_out, bsz, n_local_kv_heads,
                                    max_seq_len, s_last_dim, n_tokens, p, st);
        } else {
            dim3 grid(p.n_chunks, n_local_kv_heads, bsz), block(head_dim / 2 < 256 ? head_dim / 2 : 256);
            if (ref)
                hipLaunchKernelGGL(v_compute_generic_kernel<true>, grid, block, 0, st, first_8, mid_4, last_4,
                                   reinterpret_cast<const unsigned short *>(s), amin, partial, levels_out,
                                   n_local_kv_heads, head_dim, max_seq_len, s_last_dim, n_tokens, p.chunk_tokens,
                                   p.n_chunks);
            else
                hipLaunchKernelGGL(v_compute_generic_kernel<false>, grid, block, 0, st, first_8, mid_4, last_4,
                                   reinterpret_cast<const unsigned short *>(s), amin, partial, levels_out,
                                   n_local_kv_heads, head_dim, max_seq_len, s_last_dim, n_tokens, p.chunk_tokens,
                                   p.n_chunks);
        }
        int rc = check_launch("v_cache_compute");
        if (rc != AKV_OK) return rc;
    }
    hipLaunchKernelGGL(v_combine_kernel, dim3(bsz * n_local_kv_heads), dim3(head_dim < 256 ? head_dim : 256), 0, st,
                       partial, reinterpret_cast<unsigned short *>(o_out), head_dim, p.n_chunks);
    return check_launch("v_cache_compute(combine)");
}
