// Dense fp16 decode attention for gfx950: the baseline the split-precision path is measured against.
// Same decomposition and the same care as the AlignedKV step (16-byte loads, fp32 accumulation,
// sequence split over workgroups, deterministic combine), but every K and V element is read as a
// full fp16 value from head-major caches [bsz, heads, max_seq_len, head_dim].
// Semantics: model/Llama_AlignedKV.py:130-139 of the reference (scores / sqrt(D), fp32 softmax cast
// to fp16, probabilities @ V), with the new token appended first.
#include "akv_cores.h"

namespace akv {

__device__ __forceinline__ float d_block_reduce(float v, bool is_max, float *red) {
    v = is_max ? wave_max(v) : wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return is_max ? fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])) : ((red[0] + red[1]) + (red[2] + red[3]));
}

// acc += dot of the 8 halves in w with the 8 floats in x
__device__ __forceinline__ float dot8(const u32x4 w, const float *x, float acc) {
    acc = fmaf(lo_half_to_float(w.x), x[0], acc);
    acc = fmaf(hi_half_to_float(w.x), x[1], acc);
    acc = fmaf(lo_half_to_float(w.y), x[2], acc);
    acc = fmaf(hi_half_to_float(w.y), x[3], acc);
    acc = fmaf(lo_half_to_float(w.z), x[4], acc);
    acc = fmaf(hi_half_to_float(w.z), x[5], acc);
    acc = fmaf(lo_half_to_float(w.w), x[6], acc);
    acc = fmaf(hi_half_to_float(w.w), x[7], acc);
    return acc;
}

// K pass, head_dim 128: a token row is 256 bytes = 16 lanes x 16 bytes, a wave-wide load covers 4 tokens,
// 8 loads are in flight per iteration (32 tokens).  grid (ceil(n_tokens / (4*tokens_per_wave)), H, B).
__global__ __launch_bounds__(256) void dense_k_pass_kernel(const unsigned short *__restrict__ k_cache,
                                                           const unsigned short *__restrict__ q,
                                                           unsigned short *__restrict__ scores, int H,
                                                           int max_seq_len, int row_stride, int n_tokens,
                                                           int tokens_per_wave, float sqrt_d) {
    constexpr int D = 128;
    fetch_arguments_now(k_cache, q, scores);
    const int lane = threadIdx.x & 63, wave = wave_index();
    const int h = blockIdx.y, b = blockIdx.z, bh = b * H + h;
    const int t_begin = (blockIdx.x * 4 + wave) * tokens_per_wave;
    if (t_begin >= n_tokens) return;
    const int t_end = min(t_begin + tokens_per_wave, n_tokens);
    const int cl = lane & 15, tl = lane >> 4;
    float qf[8];
    {
        const u32x4 w = *reinterpret_cast<const u32x4 *>(q + (int64_t)bh * D + cl * 8);
        const u32 ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            qf[2 * j] = lo_half_to_float(ww[j]);
            qf[2 * j + 1] = hi_half_to_float(ww[j]);
        }
    }
    const __amdgpu_buffer_rsrc_t rK = make_rsrc(k_cache + (int64_t)bh * max_seq_len * D, (u32)n_tokens * D * 2);
    unsigned short *s_row = scores + (int64_t)bh * row_stride;
    // software pipeline: the 8 loads of the next 32 tokens are in flight while the current ones are multiplied
    auto issue = [&](u32x4 *kv, int base) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int t = base + u * 4 + tl;
            kv[u] = __builtin_amdgcn_raw_buffer_load_b128(rK, t < t_end ? t * (D * 2) + cl * 16 : kSkip, 00, kStream);
        }
    };
    auto finish = [&](const u32x4 *kv, int base) {
        float acc[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc[u] = dot8(kv[u], qf, 0.f);
        // fold the 16 lanes of a token: 8 sums -> 1 over lane bits 0..2, then bit 3
        reduce_scatter_step<8>(acc, 1);
        reduce_scatter_step<4>(acc, 2);
        reduce_scatter_step<2>(acc, 4);
        acc[0] += __shfl_xor(acc[0], 8, 64);
        const int u = ((lane & 1) ? 4 : 0) + ((lane & 2) ? 2 : 0) + ((lane & 4) ? 1 : 0);
        const int t = base + u * 4 + tl;
        // fp16 matmul result, then the fp16 division by sqrt(D) (model/Llama_AlignedKV.py:130)
        if ((lane & 8) == 0 && t < t_end)
            s_row[t] = float_to_half_bits(half_bits_to_float(float_to_half_bits(acc[0])) / sqrt_d);
    };
    u32x4 ka[8], kb[8];
    issue(ka, t_begin);
    __builtin_amdgcn_sched_barrier(0);
    for (int base = t_begin; base < t_end; base += 64) {
        issue(kb, base + 32);
        __builtin_amdgcn_sched_barrier(0);
        finish(ka, base);
        __builtin_amdgcn_sched_barrier(0);
        issue(ka, base + 64);
        __builtin_amdgcn_sched_barrier(0);
        finish(kb, base + 32);
        __builtin_amdgcn_sched_barrier(0);
    }
}

struct DenseMiddleArgs {
    const unsigned short *q, *k_new, *v_new;
    unsigned short *k_cache, *v_cache, *scores, *probs;
    int H, max_seq_len, row_stride, n_old;   // n_old tokens already cached; the new one goes to row n_old
};

// softmax over n_old + 1 scores, append of the new token.  grid (B*H), 256 threads.
__global__ __launch_bounds__(256) void dense_middle_kernel(DenseMiddleArgs a) {
    constexpr int D = 128;
    __shared__ float red[4];
    __shared__ float s_new;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bh = blockIdx.x;
    const unsigned short *qrow = a.q + (int64_t)bh * D;
    const unsigned short *knew = a.k_new + (int64_t)bh * D;
    const unsigned short *vnew = a.v_new + (int64_t)bh * D;
    unsigned short *srow = a.scores + (int64_t)bh * a.row_stride;
    unsigned short *prow = a.probs + (int64_t)bh * a.row_stride;
    const int n = a.n_old;
    if (tid < D) {
        a.k_cache[((int64_t)bh * a.max_seq_len + n) * D + tid] = knew[tid];
        a.v_cache[((int64_t)bh * a.max_seq_len + n) * D + tid] = vnew[tid];
    }
    if (wave == 0) {
        float part = 0.f;
        for (int c = lane; c < D; c += 64) part = fmaf(half_bits_to_float(knew[c]), half_bits_to_float(qrow[c]), part);
        part = wave_sum(part);
        if (lane == 0) {
            const unsigned short sc = float_to_half_bits(half_bits_to_float(float_to_half_bits(part)) / sqrtf((float)D));
            srow[n] = sc;
            s_new = half_bits_to_float(sc);
        }
    }
    __syncthreads();
    // scores of the cached tokens as 16-byte vectors; rows of up to 8192 tokens stay in registers between the passes
    constexpr int VPT = 4;
    const int nvec = n >> 3;
    const bool in_regs = nvec <= 256 * VPT;
    u32x4 sv[VPT];
    auto vec = [&](int v) -> u32x4 { return in_regs ? sv[v] : *reinterpret_cast<const u32x4 *>(srow + (tid + 256 * v) * 8); };
    const int nv = in_regs ? VPT : (nvec + 255) / 256;
    if (in_regs) {
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            const int i = tid + 256 * v;
            sv[v] = i < nvec ? *reinterpret_cast<const u32x4 *>(srow + i * 8) : (u32x4){0xfc00fc00u, 0xfc00fc00u, 0xfc00fc00u, 0xfc00fc00u};
        }
    }
    auto each = [&](auto &&f) {   // f(vector index, 8 floats) over this thread's vectors
        if (in_regs) {
#pragma unroll
            for (int v = 0; v < VPT; ++v) {
                const int i = tid + 256 * v;
                if (i < nvec) f(i, sv[v]);
            }
        } else {
            for (int v = 0; v < nv; ++v) {
                const int i = tid + 256 * v;
                if (i < nvec) f(i, *reinterpret_cast<const u32x4 *>(srow + i * 8));
            }
        }
    };
    (void)vec;
    // the tokens after the last whole vector and the new one: scalar
    const int t_tail = (nvec << 3) + tid;
    const float x_tail = t_tail < n ? half_bits_to_float(srow[t_tail]) : (t_tail == n ? s_new : -INFINITY);
    float m = x_tail;
    each([&](int, const u32x4 w) {
        const u32 ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) m = fmaxf(m, fmaxf(lo_half_to_float(ww[j]), hi_half_to_float(ww[j])));
    });
    m = d_block_reduce(m, true, red);
    float sum = t_tail <= n ? expf(x_tail - m) : 0.f;
    each([&](int, const u32x4 w) {
        const u32 ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) sum += expf(lo_half_to_float(ww[j]) - m) + expf(hi_half_to_float(ww[j]) - m);
    });
    sum = d_block_reduce(sum, false, red);
    const float rsum = 1.0f / sum;
    each([&](int i, const u32x4 w) {
        const u32 ww[4] = {w.x, w.y, w.z, w.w};
        u32 o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            o[j] = (u32)float_to_half_bits(div_by(expf(lo_half_to_float(ww[j]) - m), sum, rsum)) |
                   ((u32)float_to_half_bits(div_by(expf(hi_half_to_float(ww[j]) - m), sum, rsum)) << 16);
        *reinterpret_cast<u32x4 *>(prow + i * 8) = (u32x4){o[0], o[1], o[2], o[3]};
    });
    if (t_tail <= n) prow[t_tail] = float_to_half_bits(div_by(expf(x_tail - m), sum, rsum));
}

// V pass, head_dim 128: lane = 8 channels of one token, 4 tokens per wave-wide load, 8 loads in flight.
// grid (n_chunks, H, B), 256 threads; partial fp32 [B*H, n_chunks, D].
__global__ __launch_bounds__(256) void dense_v_pass_kernel(const unsigned short *__restrict__ v_cache,
                                                           const unsigned short *__restrict__ probs,
                                                           float *__restrict__ partial, int H, int max_seq_len,
                                                           int row_stride, int n_tokens, int tokens_per_wave,
                                                           int n_chunks) {
    constexpr int D = 128;
    fetch_arguments_now(v_cache, probs, partial);
    __shared__ float wave_part[4][D];
    const int lane = threadIdx.x & 63, wave = wave_index();
    const int chunk = blockIdx.x, h = blockIdx.y, b = blockIdx.z, bh = b * H + h;
    const int t_begin = (chunk * 4 + wave) * tokens_per_wave;
    const int t_end = min(t_begin + tokens_per_wave, n_tokens);
    const int cl = lane & 15, tl = lane >> 4;
    const __amdgpu_buffer_rsrc_t rV = make_rsrc(v_cache + (int64_t)bh * max_seq_len * D, (u32)n_tokens * D * 2);
    const __amdgpu_buffer_rsrc_t rS = make_rsrc(probs + (int64_t)bh * row_stride, (u32)n_tokens * 2);
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
    auto issue = [&](u32x4 *vv, u32 *sb, int base) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int t = base + u * 4 + tl;
            vv[u] = __builtin_amdgcn_raw_buffer_load_b128(rV, t < t_end ? t * (D * 2) + cl * 16 : kSkip, 00, kStream);
            sb[u] = (u32)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(rS, t < t_end ? t * 2 : kSkip, 0, 0);
        }
    };
    auto finish = [&](const u32x4 *vv, const u32 *sb) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const float sf = half_bits_to_float(sb[u]);
            acc[0] = fmaf(lo_half_to_float(vv[u].x), sf, acc[0]);
            acc[1] = fmaf(hi_half_to_float(vv[u].x), sf, acc[1]);
            acc[2] = fmaf(lo_half_to_float(vv[u].y), sf, acc[2]);
            acc[3] = fmaf(hi_half_to_float(vv[u].y), sf, acc[3]);
            acc[4] = fmaf(lo_half_to_float(vv[u].z), sf, acc[4]);
            acc[5] = fmaf(hi_half_to_float(vv[u].z), sf, acc[5]);
            acc[6] = fmaf(lo_half_to_float(vv[u].w), sf, acc[6]);
            acc[7] = fmaf(hi_half_to_float(vv[u].w), sf, acc[7]);
        }
    };
    // software pipeline: the next 32 token rows are in flight while the current ones are multiplied
    u32x4 va[8], vb[8];
    u32 sa[8], sbb[8];
    issue(va, sa, t_begin);
    __builtin_amdgcn_sched_barrier(0);
    for (int base = t_begin; base < t_end; base += 64) {
        issue(vb, sbb, base + 32);
        __builtin_amdgcn_sched_barrier(0);
        finish(va, sa);
        __builtin_amdgcn_sched_barrier(0);
        issue(va, sa, base + 64);
        __builtin_amdgcn_sched_barrier(0);
        finish(vb, sbb);
        __builtin_amdgcn_sched_barrier(0);
    }
    // fold the 4 token lanes (lane bits 4, 5): 8 sums -> 2 per lane
    int ch = cl * 8;
    reduce_scatter_step<8>(acc, 32);
    ch += (lane & 32) ? 4 : 0;
    reduce_scatter_step<4>(acc, 16);
    ch += (lane & 16) ? 2 : 0;
    wave_part[wave][ch] = acc[0];
    wave_part[wave][ch + 1] = acc[1];
    __syncthreads();
    if (threadIdx.x < D) {
        const int d = threadIdx.x;
        partial[((int64_t)bh * n_chunks + chunk) * D + d] =
            (wave_part[0][d] + wave_part[1][d]) + (wave_part[2][d] + wave_part[3][d]);
    }
}

__global__ void dense_combine_kernel(const float *__restrict__ partial, unsigned short *__restrict__ out, int D, int n_chunks) {
    const int bh = blockIdx.x;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        float acc = 0.f;
        for (int c = 0; c < n_chunks; ++c) acc += partial[((int64_t)bh * n_chunks + c) * D + d];
        out[(int64_t)bh * D + d] = float_to_half_bits(acc);
    }
}

static int dense_tokens_per_wave(int B, int H, int n_tokens) {
    int tpw = 32;
    while (tpw < 256 && (int64_t)B * H * ((n_tokens + 8 * tpw - 1) / (8 * tpw)) >= 2048) tpw *= 2;
    return tpw;
}

}  // namespace akv

using namespace akv;

extern "C" size_t akv_dense_decode_step_workspace_bytes(int bsz, int n_heads, int head_dim, int max_seq_len) {
    if (bsz <= 0 || n_heads <= 0 || head_dim <= 0 || max_seq_len <= 0) return 0;
    size_t chunks = ((size_t)max_seq_len + 127) / 128;
    return (((size_t)bsz * n_heads * chunks * head_dim * sizeof(float)) + 255) & ~(size_t)255;
}

extern "C" int akv_dense_decode_step(uint8_t *k_cache, uint8_t *v_cache, const uint8_t *q, const uint8_t *k_new,
                                     const uint8_t *v_new, uint8_t *out, uint8_t *scores, uint8_t *probs,
                                     int row_stride, void *workspace, size_t workspace_bytes, int bsz, int n_heads,
                                     int max_seq_len, int head_dim, int cur_len, akv_stream_t stream) {
    AKV_REQUIRE(k_cache && v_cache && q && k_new && v_new && out && scores && probs && workspace,
                "dense_decode_step: null pointer");
    AKV_REQUIRE(head_dim == 128, "dense_decode_step: the dense baseline is written for head_dim 128 (got %d)", head_dim);
    AKV_REQUIRE(bsz > 0 && n_heads > 0 && bsz <= 65535 && n_heads <= 65535, "dense_decode_step: bad bsz/heads");
    AKV_REQUIRE(cur_len >= 0 && cur_len + 1 <= max_seq_len, "dense_decode_step: cache full (%d of %d)", cur_len, max_seq_len);
    AKV_REQUIRE(row_stride >= cur_len + 1 && row_stride % 8 == 0 && ((uintptr_t)scores & 15) == 0 && ((uintptr_t)probs & 15) == 0,
                "dense_decode_step: row_stride %d must be a multiple of 8 and >= %d, scores/probs 16-byte aligned", row_stride,
                cur_len + 1);
    AKV_REQUIRE((int64_t)max_seq_len * head_dim * 2 < (int64_t)1 << 31, "dense_decode_step: one (batch, head) slice must stay below 2 GiB");
    AKV_REQUIRE(workspace_bytes >= akv_dense_decode_step_workspace_bytes(bsz, n_heads, head_dim, max_seq_len),
                "dense_decode_step: workspace too small");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const unsigned short *q16 = reinterpret_cast<const unsigned short *>(q);
    unsigned short *kc = reinterpret_cast<unsigned short *>(k_cache), *vc = reinterpret_cast<unsigned short *>(v_cache);
    unsigned short *s16 = reinterpret_cast<unsigned short *>(scores), *p16 = reinterpret_cast<unsigned short *>(probs);
    float *partial = static_cast<float *>(workspace);
    const float sqrt_d = sqrtf((float)head_dim);
    const int n_old = cur_len, total = cur_len + 1;
    if (n_old > 0) {
        const int tpw = dense_tokens_per_wave(bsz, n_heads, n_old);
        hipLaunchKernelGGL(dense_k_pass_kernel, dim3((n_old + 4 * tpw - 1) / (4 * tpw), n_heads, bsz), dim3(256), 0, st,
                           kc, q16, s16, n_heads, max_seq_len, row_stride, n_old, tpw, sqrt_d);
        int rc = check_launch("dense_decode_step(k_pass)");
        if (rc != AKV_OK) return rc;
    }
    DenseMiddleArgs ma;
    ma.q = q16;
    ma.k_new = reinterpret_cast<const unsigned short *>(k_new);
    ma.v_new = reinterpret_cast<const unsigned short *>(v_new);
    ma.k_cache = kc; ma.v_cache = vc; ma.scores = s16; ma.probs = p16;
    ma.H = n_heads; ma.max_seq_len = max_seq_len; ma.row_stride = row_stride; ma.n_old = n_old;
    hipLaunchKernelGGL(dense_middle_kernel, dim3(bsz * n_heads), dim3(256), 0, st, ma);
    int rc = check_launch("dense_decode_step(middle)");
    if (rc != AKV_OK) return rc;
    int tpw = dense_tokens_per_wave(bsz, n_heads, total);
    if (tpw < 32) tpw = 32;
    const int n_chunks = (total + 4 * tpw - 1) / (4 * tpw);
    hipLaunchKernelGGL(dense_v_pass_kernel, dim3(n_chunks, n_heads, bsz), dim3(256), 0, st, vc, p16, partial, n_heads,
                       max_seq_len, row_stride, total, tpw, n_chunks);
    rc = check_launch("dense_decode_step(v_pass)");
    if (rc != AKV_OK) return rc;
    hipLaunchKernelGGL(dense_combine_kernel, dim3(bsz * n_heads), dim3(128), 0, st, partial,
                       reinterpret_cast<unsigned short *>(out), head_dim, n_chunks);
    return check_launch("dense_decode_step(combine)");
}
