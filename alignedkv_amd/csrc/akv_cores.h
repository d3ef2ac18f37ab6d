// Wave-level cores of the two streaming kernels, shared by the stand-alone ops (akv_k.hip,
// akv_v.hip) and the fused decode step (akv_fused.hip).
#pragma once

#include "akv_common.h"

#include <stdlib.h>

namespace akv {

template <int N>
__device__ __forceinline__ void reduce_scatter_step(float *a, int lane_mask) {
    // N partial sums per lane -> N/2: the lane keeps one half and receives the partner's sums of
    // that half.  After the step a[i] belongs to original index i + (lane & lane_mask ? N/2 : 0).
    const bool up = (threadIdx.x & lane_mask) != 0;
#pragma unroll
    for (int i = 0; i < N / 2; ++i) {
        float send = up ? a[i] : a[i + N / 2];
        float keep = up ? a[i + N / 2] : a[i];
        a[i] = keep + __shfl_xor(send, lane_mask, 64);
    }
}

// ------------------------------------------------------------------------------------------------
// K: scores of blocks [first_blk, end_blk) of one (batch, head), d_block == 64.
//   f8/m4/l4 point at block 0 of this (batch, head); n_blocks bounds the buffer resources.
//   Lane layout: load group g (16 channels) x lane -> channel g*16 + lane/4, slots (lane&3)*16..+16.
//   qf[g]: q of the lane's channel in group g; bit g of need_mid / need_last: fetch that plane.
//   s_row: fp16 scores of this (batch, head); s_row[blk*64 + slot] = fp16(dot * scale).
// ------------------------------------------------------------------------------------------------
template <int D>
__device__ __forceinline__ void k_score_blocks(const uint8_t *f8, const uint8_t *m4, const uint8_t *l4, int n_blocks,
                                               int first_blk, int end_blk, const float *qf, u32 need_mid,
                                               u32 need_last, unsigned short *s_row, float scale) {
    constexpr int CB = 64;
    constexpr int NG = D / 16;
    constexpr int GC = NG < 8 ? NG : 8;   // load groups in flight at a time
    const int lane = threadIdx.x & 63;
    const __amdgpu_buffer_rsrc_t rH = make_rsrc(f8, (u32)n_blocks * (D * CB));
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(m4, (u32)n_blocks * (D * CB / 2));
    const __amdgpu_buffer_rsrc_t rL = make_rsrc(l4, (u32)n_blocks * (D * CB / 2));
    for (int blk = first_blk; blk < end_blk; ++blk) {
        float acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
        for (int g0 = 0; g0 < NG; g0 += GC) {
            u32x4 hv[GC];
            u32x2 mv[GC], lv[GC];
#pragma unroll
            for (int g = 0; g < GC; ++g) {
                const int gg = g0 + g;
                hv[g] = __builtin_amdgcn_raw_buffer_load_b128(rH, blk * (D * CB) + gg * 1024 + lane * 16, 0, 0);
                int mo = ((need_mid >> gg) & 1u) ? blk * (D * CB / 2) + gg * 512 + lane * 8 : kSkip;
                int lo = ((need_last >> gg) & 1u) ? blk * (D * CB / 2) + gg * 512 + lane * 8 : kSkip;
                mv[g] = __builtin_amdgcn_raw_buffer_load_b64(rM, mo, 0, 0);
                lv[g] = __builtin_amdgcn_raw_buffer_load_b64(rL, lo, 0, 0);
            }
#pragma unroll
            for (int g = 0; g < GC; ++g) {
                const int gg = g0 + g;
                const u32 cm = ((need_mid >> gg) & 1u) ? 0u : 0x88888888u;                                 // level 2
                const u32 cl = (((need_mid >> gg) & 1u) && !((need_last >> gg) & 1u)) ? 0x88888888u : 0u;  // level 1
                fma8(acc, hv[g].x, hv[g].y, mv[g].x | cm, lv[g].x | cl, qf[gg]);
                fma8(acc + 8, hv[g].z, hv[g].w, mv[g].y | cm, lv[g].y | cl, qf[gg]);
            }
        }
        // acc[i]: partial score of slot (lane&3)*16 + i over this lane's channels
        reduce_scatter_step<16>(acc, 32);
        reduce_scatter_step<8>(acc, 16);
        reduce_scatter_step<4>(acc, 8);
        reduce_scatter_step<2>(acc, 4);
        const int slot = (lane & 3) * 16 + ((lane & 32) ? 8 : 0) + ((lane & 16) ? 4 : 0) + ((lane & 8) ? 2 : 0) +
                         ((lane & 4) ? 1 : 0);
        s_row[blk * CB + slot] = float_to_half_bits(acc[0] * scale);
    }
}

// ------------------------------------------------------------------------------------------------
// V: one wave accumulates tokens [t_begin, t_end) of one (batch, head) into acc[16].
//   f8/m4/l4 point at token 0 of this (batch, head); n_tokens bounds the buffer resources.
//   Lane layout: lane -> token (lane / (D/16)) of each wave-wide load, channels (lane % (D/16))*16..+16.
//   s_row: fp16 probabilities of this (batch, head).  levels_row (may be null): level per token.
// ------------------------------------------------------------------------------------------------
template <int D, bool REF, int NIT>
__device__ __forceinline__ void v_accumulate(const uint8_t *f8, const uint8_t *m4, const uint8_t *l4, int n_tokens,
                                             const unsigned short *s_row, unsigned char amin, int t_begin, int t_end,
                                             float *acc, uint8_t *levels_row) {
    constexpr int LPR = D / 16;            // lanes per token row
    constexpr int TPL = 64 / LPR;          // token rows per wave-wide load
    constexpr int U = LPR < 8 ? LPR : 8;   // loads in flight per iteration
    const int lane = threadIdx.x & 63;
    const int tl = lane / LPR, cl = lane % LPR;
    const __amdgpu_buffer_rsrc_t rH = make_rsrc(f8, (u32)n_tokens * D);
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(m4, (u32)n_tokens * (D / 2));
    const __amdgpu_buffer_rsrc_t rL = make_rsrc(l4, (u32)n_tokens * (D / 2));
    const __amdgpu_buffer_rsrc_t rS = make_rsrc(s_row, (u32)n_tokens * 2);
    // The probabilities of all the wave's tokens first: the fetch level of a token depends on its
    // probability, and a load per iteration would put a memory round trip in front of every batch.
    u32 sb[NIT][U];
#pragma unroll
    for (int it = 0; it < NIT; ++it)
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int t = t_begin + (it * U + u) * TPL + tl;
            sb[it][u] = (u32)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(rS, t < t_end ? t * 2 : kSkip, 0, 0);
        }
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
        const int base = t_begin + it * U * TPL;
        if (base >= t_end) break;
        u32x4 hv[U];
        u32x2 mv[U], lv[U];
        // the high-byte rows do not depend on the level: issue them before the probabilities are looked at
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int t = base + u * TPL + tl;
            hv[u] = __builtin_amdgcn_raw_buffer_load_b128(rH, t < t_end ? t * D + cl * 16 : kSkip, 0, 0);
        }
        u32 cm[U], cl_[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int t = base + u * TPL + tl;
            const bool valid = t < t_end;
            const int level = REF ? 0 : v_level(amin, (unsigned short)sb[it][u]);
            mv[u] = __builtin_amdgcn_raw_buffer_load_b64(rM, (valid && level < 2) ? t * (D / 2) + cl * 8 : kSkip, 0, 0);
            lv[u] = __builtin_amdgcn_raw_buffer_load_b64(rL, (valid && level == 0) ? t * (D / 2) + cl * 8 : kSkip, 0, 0);
            cm[u] = level == 2 ? 0x88888888u : 0u;
            cl_[u] = level == 1 ? 0x88888888u : 0u;
            if (levels_row != nullptr && valid && cl == 0) levels_row[t] = (uint8_t)level;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float sf = half_bits_to_float(sb[it][u]);
            fma8(acc, hv[u].x, hv[u].y, mv[u].x | cm[u], lv[u].x | cl_[u], sf);
            fma8(acc + 8, hv[u].z, hv[u].w, mv[u].y | cm[u], lv[u].y | cl_[u], sf);
        }
    }
}

// Folds the token lanes of a wave together and adds the 4 waves of the workgroup:
// out[d] (d < D) = sum over all 256 lanes of their acc for channel d.  wave_part: LDS [4][D].
template <int D>
__device__ __forceinline__ void v_fold_workgroup(float *acc, float (*wave_part)[D], float *out) {
    constexpr int LPR = D / 16;
    constexpr int NV = LPR == 16 ? 4 : (LPR == 8 ? 2 : 1);   // sums left per lane
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int ch = (lane % LPR) * 16;
    reduce_scatter_step<16>(acc, 32);
    ch += (lane & 32) ? 8 : 0;
    reduce_scatter_step<8>(acc, 16);
    ch += (lane & 16) ? 4 : 0;
    if constexpr (LPR <= 8) {
        reduce_scatter_step<4>(acc, 8);
        ch += (lane & 8) ? 2 : 0;
    }
    if constexpr (LPR <= 4) {
        reduce_scatter_step<2>(acc, 4);
        ch += (lane & 4) ? 1 : 0;
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) wave_part[wave][ch + i] = acc[i];
    __syncthreads();
    for (int d = threadIdx.x; d < D; d += 256)
        out[d] = (wave_part[0][d] + wave_part[1][d]) + (wave_part[2][d] + wave_part[3][d]);
}

// Split of the sequence over workgroups for the V pass (shared by the op and the fused step).
struct VPlan {
    bool tuned;
    int iters_per_wave;    // tuned kernel: 1, 2 or 4 batches of 64 (32 for head_dim 256) tokens per wave
    int tokens_per_wave;
    int chunk_tokens;      // tokens per workgroup
    int n_chunks;
};

inline VPlan v_plan(int B, int H, int D, int n_tokens) {
    VPlan p;
    p.tuned = (D == 64 || D == 128 || D == 256);
    if (p.tuned) {
        const int iter_tokens = D == 256 ? 32 : 64;
        int k = 1;   // iterations per wave: 1, 2 or 4
        while (k < 4 && (int64_t)B * H * ((n_tokens + 4 * iter_tokens * k * 2 - 1) / (4 * iter_tokens * k * 2)) >= 2048) k *= 2;
        if (const char *e = getenv("AKV_TUNE_V_ITERS")) k = atoi(e) == 4 ? 4 : (atoi(e) == 2 ? 2 : 1);
        p.iters_per_wave = k;
        p.tokens_per_wave = iter_tokens * k;
        p.chunk_tokens = 4 * p.tokens_per_wave;
    } else {
        p.iters_per_wave = 0;
        p.tokens_per_wave = 0;
        p.chunk_tokens = 256;
    }
    p.n_chunks = n_tokens > 0 ? (n_tokens + p.chunk_tokens - 1) / p.chunk_tokens : 0;
    return p;
}

inline int k_blocks_per_wave(int B, int H, int n_blocks) {
    // enough waves to fill 256 CUs several times over, a few blocks per wave to amortise set-up
    int bpw = 1;
    while (bpw < 4 && (int64_t)B * H * ((n_blocks + bpw * 2 - 1) / (bpw * 2)) >= 8192) bpw *= 2;
    if (const char *e = getenv("AKV_TUNE_K_BPW")) bpw = atoi(e) > 0 ? atoi(e) : bpw;
    return bpw;
}

}  // namespace akv
