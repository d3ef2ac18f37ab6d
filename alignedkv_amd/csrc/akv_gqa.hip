// Grouped-query K and V passes of the fused decode step: one workgroup streams a chunk of a KV head's planes
// ONCE and multiplies it with GH query heads of that KV head's group.
//
// The reference keeps one KV head per query head (model/KVCache_AlignedKV.py:32 asserts it), so its fetch level
// is per query head: K per (batch, head, channel) (extension/csrc/K_cache.cu:211,249-252), V per (batch, head,
// token) (extension/csrc/V_cache.cu:195-197,250-253).  Here every query head keeps exactly its own levels: a
// plane row is fetched when ANY head of the group needs it, and each head substitutes the reference's constants
// (0x8 / 0x80) for the planes ITS level skips, as a (keep, put) mask pair on the fetched low bytes.  Results are
// those of the per-head kernels on repeated planes; HBM traffic is that of the KV heads.
#include "akv_step.h"

namespace akv {

// ------------------------------------------------------------------------------------------------
// K pass.  grid (ceil(n_blocks / (4*blocks_per_wave)), Hkv * G/GH, B), 256 threads.
// ------------------------------------------------------------------------------------------------
template <int HG, int NG, int GH>
__device__ __forceinline__ void k_compute_half_group(float (*acc)[16], const KHalfTile<HG> &t, int g0,
                                                     const float (*qf)[NG], const u32 (*keep)[NG], const u32 (*put)[NG]) {
#pragma unroll
    for (int g = 0; g < HG; ++g) {
        const int gg = g0 + g;
        u32 E0, O0, E1, O1;
        split_even_odd(t.m[g].x, t.l[g].x, E0, O0);
        split_even_odd(t.m[g].y, t.l[g].y, E1, O1);
#pragma unroll
        for (int h = 0; h < GH; ++h) {
            const u32 a = keep[h][gg], c = put[h][gg];
            fma8_even_odd(acc[h], t.h[g].x, t.h[g].y, (E0 & a) | c, (O0 & a) | c, qf[h][gg]);
            fma8_even_odd(acc[h] + 8, t.h[g].z, t.h[g].w, (E1 & a) | c, (O1 & a) | c, qf[h][gg]);
        }
    }
}

template <int D, bool REF, int GH>
__global__ __launch_bounds__(256) void group_k_pass_kernel(
    const uint8_t *__restrict__ first_8, const uint8_t *__restrict__ mid_4, const uint8_t *__restrict__ last_4,
    const uint8_t *__restrict__ kcm, const unsigned short *__restrict__ q, const unsigned short *__restrict__ k_new,
    unsigned short *__restrict__ scores, uint8_t *__restrict__ levels_out, StepGeom geo, int blocks_per_wave,
    float scale) {
    constexpr int CB = 64;
    constexpr int NG = D / 16;
    constexpr int HG = NG / 2;
    const int lane = threadIdx.x & 63, wave = wave_index();
    int chunk, by, b;
    if (!step_block(geo, chunk, by, b)) return;
    const int n_sub = geo.G / GH;
    const int hkv = by / n_sub;
    const int hq0 = hkv * geo.G + (by - hkv * n_sub) * GH;   // first query head of this workgroup
    const int bh_kv = b * geo.Hkv + hkv;
    const int64_t bh0 = (int64_t)b * geo.Hq + hq0;
    int R, nrest;
    seq_state(geo, b, R, nrest);
    const int n_blocks = R / CB;
    const int first_blk = (chunk * 4 + wave) * blocks_per_wave;
    const int end_blk = min(first_blk + blocks_per_wave, n_blocks);
    // the grid covers the longest sequence: waves past the end of this one leave before the set-up (no barrier
    // in this kernel); the wave that records the levels stays
    if (first_blk >= n_blocks && !(levels_out != nullptr && chunk == 0 && wave == 0)) return;

    const int64_t plane_off = (int64_t)bh_kv * geo.n_max_blocks * (D * (CB / 2));
    const uint8_t *f8 = first_8 + plane_off * 2, *m4 = mid_4 + plane_off, *l4 = last_4 + plane_off;
    KHalfTile<HG> ta;
    k_prefetch_first<D>(ta, f8, n_blocks, first_blk);

    // per query head: q of the lane's channels and the (keep, put) masks of its fetch levels
    float qf[GH][NG];
    u32 keep[GH][NG], put[GH][NG];
    u32 need_mid = 0, need_last = 0;
    u32 cmax[NG];
#pragma unroll
    for (int g = 0; g < NG; ++g) {
        const int c = g * 16 + (lane >> 2);
        // column max including the token appended by this step
        cmax[g] = max((u32)kcm[(int64_t)bh_kv * D + c], exp_field(k_new[(int64_t)bh_kv * D + c]));
    }
#pragma unroll
    for (int h = 0; h < GH; ++h) {
        u32 esum[NG];
        u32 mx = 0;
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            const u32 qb = q[(bh0 + h) * D + g * 16 + (lane >> 2)];
            qf[h][g] = half_bits_to_float(qb);
            esum[g] = (exp_field(qb) + cmax[g]) & 0xffu;
            mx = max(mx, esum[g]);
        }
        mx = quads_max_u32(mx);
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            const int lv = REF ? 0 : k_level((unsigned char)mx, (unsigned char)esum[g]);
            level_masks(lv, keep[h][g], put[h][g]);
            need_mid |= (lv < 2 ? 1u : 0u) << g;      // a plane row is fetched if any head of the group reads it
            need_last |= (lv == 0 ? 1u : 0u) << g;
            if (levels_out != nullptr && chunk == 0 && wave == 0 && (lane & 3) == 0)
                levels_out[(bh0 + h) * D + g * 16 + (lane >> 2)] = (uint8_t)lv;
        }
    }

    const __amdgpu_buffer_rsrc_t rH = make_rsrc(f8, (u32)n_blocks * (D * CB));
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(m4, (u32)n_blocks * (D * CB / 2));
    const __amdgpu_buffer_rsrc_t rL = make_rsrc(l4, (u32)n_blocks * (D * CB / 2));
    const int slot = (lane & 3) * 16 + ((lane & 32) ? 8 : 0) + ((lane & 16) ? 4 : 0) + ((lane & 8) ? 2 : 0) +
                     ((lane & 4) ? 1 : 0);
    // software pipeline over half blocks, as k_score_blocks
    KHalfTile<HG> tb;
    k_issue_half_ml<D, HG>(ta, rM, rL, first_blk, 0, need_mid, need_last);
    __builtin_amdgcn_sched_barrier(0);
    for (int blk = first_blk; blk < end_blk; ++blk) {
        float acc[GH][16];
#pragma unroll
        for (int h = 0; h < GH; ++h)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[h][i] = 0.f;
        k_issue_half<D, HG>(tb, rH, rM, rL, blk, HG, need_mid, need_last);
        __builtin_amdgcn_sched_barrier(0);
        k_compute_half_group<HG, NG, GH>(acc, ta, 0, qf, keep, put);
        __builtin_amdgcn_sched_barrier(0);
        k_issue_half<D, HG>(ta, rH, rM, rL, blk + 1 < end_blk ? blk + 1 : n_blocks, 0, need_mid, need_last);
        __builtin_amdgcn_sched_barrier(0);
        k_compute_half_group<HG, NG, GH>(acc, tb, HG, qf, keep, put);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int h = 0; h < GH; ++h) {
            reduce_scatter_step<16>(acc[h], 32);
            reduce_scatter_step<8>(acc[h], 16);
            reduce_scatter_step<4>(acc[h], 8);
            reduce_scatter_step<2>(acc[h], 4);
            const __amdgpu_buffer_rsrc_t rS = make_rsrc(scores + (bh0 + h) * geo.row_stride, (u32)n_blocks * CB * 2);
            store_u16_device(rS, (blk * CB + slot) * 2, float_to_half_bits(acc[h][0] * scale));
        }
    }
}

// ------------------------------------------------------------------------------------------------
// V pass.  grid (n_chunks, Hkv * G/GH, B), 256 threads; a wave walks tokens_per_wave tokens in steps of
// 2 half tiles (64 tokens; 32 for head_dim 256).
// ------------------------------------------------------------------------------------------------
template <int D, bool REF, int GH>
struct VGroupProbs {   // probabilities of the tokens of two half tiles, per query head
    static constexpr int U = (D / 16 < 8 ? D / 16 : 8);
    u32 s[GH][U];
};

template <int D, bool REF, int GH>
__device__ __forceinline__ void v_group_load_probs(VGroupProbs<D, REF, GH> &p, const __amdgpu_buffer_rsrc_t *rS, int base,
                                                   int t_end) {
    constexpr int LPR = D / 16, TPL = 64 / LPR, U = VGroupProbs<D, REF, GH>::U;
    const int tl = (threadIdx.x & 63) / LPR;
#pragma unroll
    for (int h = 0; h < GH; ++h)
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int t = base + u * TPL + tl;
            p.s[h][u] = (u32)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(rS[h], t < t_end ? t * 2 : kSkip, 0, 0);
        }
}

// requests half tile `half` (0/1) of the 2-half-tile step that starts at token `base`
template <int D, bool REF, int GH, int HV>
__device__ __forceinline__ void v_group_issue(VHalfTile<HV> &t, const __amdgpu_buffer_rsrc_t rH,
                                              const __amdgpu_buffer_rsrc_t rM, const __amdgpu_buffer_rsrc_t rL, int base,
                                              int half, int t_end, const VGroupProbs<D, REF, GH> &p, const unsigned char *amin) {
    constexpr int LPR = D / 16, TPL = 64 / LPR;
    const int lane = threadIdx.x & 63;
    const int tl = lane / LPR, cl = lane % LPR;
    v_issue_half_h<D, HV>(t, rH, base + half * HV * TPL, t_end);
#pragma unroll
    for (int u = 0; u < HV; ++u) {
        const int tok = base + (half * HV + u) * TPL + tl;
        const bool valid = tok < t_end;
        int level = 2;   // finest level any head of the group asks for
#pragma unroll
        for (int h = 0; h < GH; ++h) level = min(level, REF ? 0 : v_level(amin[h], (unsigned short)p.s[h][half * HV + u]));
        t.m[u] = __builtin_amdgcn_raw_buffer_load_b64(rM, (valid && level < 2) ? tok * (D / 2) + cl * 8 : kSkip, 00, kStream);
        t.l[u] = __builtin_amdgcn_raw_buffer_load_b64(rL, (valid && level == 0) ? tok * (D / 2) + cl * 8 : kSkip, 00, kStream);
    }
}

template <int D, bool REF, int GH, int HV>
__device__ __forceinline__ void v_group_compute(float (*acc)[16], const VHalfTile<HV> &t, int half,
                                                const VGroupProbs<D, REF, GH> &p, const unsigned char *amin) {
#pragma unroll
    for (int u = 0; u < HV; ++u) {
        u32 E0, O0, E1, O1;
        split_even_odd(t.m[u].x, t.l[u].x, E0, O0);
        split_even_odd(t.m[u].y, t.l[u].y, E1, O1);
#pragma unroll
        for (int h = 0; h < GH; ++h) {
            const u32 sb = p.s[h][half * HV + u];
            u32 a, c;
            level_masks(REF ? 0 : v_level(amin[h], (unsigned short)sb), a, c);
            const float sf = half_bits_to_float(sb);
            fma8_even_odd(acc[h], t.h[u].x, t.h[u].y, (E0 & a) | c, (O0 & a) | c, sf);
            fma8_even_odd(acc[h] + 8, t.h[u].z, t.h[u].w, (E1 & a) | c, (O1 & a) | c, sf);
        }
    }
}

template <int GH>
__device__ __forceinline__ void pin_group(float (*acc)[16]) {
#pragma unroll
    for (int h = 0; h < GH; ++h) pin_accumulators(acc[h]);
}

template <int D, bool REF, int GH>
__global__ __launch_bounds__(256) void group_v_pass_kernel(
    const uint8_t *__restrict__ first_8, const uint8_t *__restrict__ mid_4, const uint8_t *__restrict__ last_4,
    const unsigned short *__restrict__ probs, const uint8_t *__restrict__ amin_u8, float *__restrict__ partial,
    uint8_t *__restrict__ levels_out, int levels_stride, uint8_t *__restrict__ amin_out, StepGeom geo,
    int tokens_per_wave, int n_chunks) {
    constexpr int LPR = D / 16, TPL = 64 / LPR;
    constexpr int U = VGroupProbs<D, REF, GH>::U, HV = U / 2;
    constexpr int ST = U * TPL;               // tokens per step of two half tiles
    __shared__ float wave_part[4][D];
    const int lane = threadIdx.x & 63, wave = wave_index();
    int chunk, by, b;
    if (!step_block(geo, chunk, by, b)) return;
    const int n_sub = geo.G / GH;
    const int hkv = by / n_sub;
    const int hq0 = hkv * geo.G + (by - hkv * n_sub) * GH;
    const int bh_kv = b * geo.Hkv + hkv;
    const int64_t bh0 = (int64_t)b * geo.Hq + hq0;
    int n_tokens, nrest;
    seq_state(geo, b, n_tokens, nrest);
    const int t_begin = (chunk * 4 + wave) * tokens_per_wave;
    const int t_end = min(t_begin + tokens_per_wave, n_tokens);
    if (chunk * 4 * tokens_per_wave >= n_tokens && chunk > 0) {   // (cannot happen with a task map)
        // the grid covers the longest sequence: a workgroup past the end of this one only clears its partial sums
        for (int i = threadIdx.x; i < GH * D; i += 256) partial[((bh0 + i / D) * n_chunks + chunk) * D + i % D] = 0.f;
        return;
    }
    const int64_t row0 = (int64_t)bh_kv * geo.max_seq_len;
    const __amdgpu_buffer_rsrc_t rH = make_rsrc(first_8 + row0 * D, (u32)n_tokens * D);
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(mid_4 + row0 * (D / 2), (u32)n_tokens * (D / 2));
    const __amdgpu_buffer_rsrc_t rL = make_rsrc(last_4 + row0 * (D / 2), (u32)n_tokens * (D / 2));
    __amdgpu_buffer_rsrc_t rS[GH];
    unsigned char amin[GH];
#pragma unroll
    for (int h = 0; h < GH; ++h) {
        rS[h] = make_rsrc(probs + (bh0 + h) * geo.row_stride, (u32)n_tokens * 2);
        amin[h] = REF ? 0 : amin_u8[bh0 + h];
        if (!REF && amin_out != nullptr && chunk == 0 && threadIdx.x == 0) amin_out[bh0 + h] = amin[h];
    }
    float acc[GH][16];
#pragma unroll
    for (int h = 0; h < GH; ++h)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[h][i] = 0.f;

    // Pipeline: while a half tile is multiplied the next one is in flight; the probabilities of a step are
    // requested one step ahead (and before the tile loads of that phase, so that waiting for them does not
    // wait for a tile).
    VGroupProbs<D, REF, GH> pc, pn;
    VHalfTile<HV> ta, tb;
    v_group_load_probs<D, REF, GH>(pc, rS, t_begin, t_end);
    v_group_issue<D, REF, GH, HV>(ta, rH, rM, rL, t_begin, 0, t_end, pc, amin);
    __builtin_amdgcn_sched_barrier(0);
    for (int base = t_begin; base < t_end; base += ST) {
        const int next = base + ST < t_end ? base + ST : t_end;   // == t_end: every load of the look-ahead is skipped
        v_group_load_probs<D, REF, GH>(pn, rS, next, t_end);
        v_group_issue<D, REF, GH, HV>(tb, rH, rM, rL, base, 1, t_end, pc, amin);
        __builtin_amdgcn_sched_barrier(0);
        v_group_compute<D, REF, GH, HV>(acc, ta, 0, pc, amin);
        pin_group<GH>(acc);
        __builtin_amdgcn_sched_barrier(0);
        v_group_issue<D, REF, GH, HV>(ta, rH, rM, rL, next, 0, t_end, pn, amin);
        __builtin_amdgcn_sched_barrier(0);
        v_group_compute<D, REF, GH, HV>(acc, tb, 1, pc, amin);
        pin_group<GH>(acc);
        __builtin_amdgcn_sched_barrier(0);
        pc = pn;
    }
    // optional record of the levels, outside the pipeline
    if (levels_out != nullptr) {
        for (int t = t_begin + lane; t < t_end; t += 64)
#pragma unroll
            for (int h = 0; h < GH; ++h)
                levels_out[(bh0 + h) * levels_stride + t] =
                    (uint8_t)(REF ? 0 : v_level(amin[h], probs[(bh0 + h) * geo.row_stride + t]));
    }
#pragma unroll
    for (int h = 0; h < GH; ++h) {
        if (h) __syncthreads();      // wave_part is reused
        v_fold_workgroup<D>(acc[h], wave_part, partial + ((bh0 + h) * n_chunks + chunk) * D);
    }
}

// ---- host ------------------------------------------------------------------------------------------
int group_heads(int G) {
    return G % 4 == 0 ? 4 : (G % 2 == 0 ? 2 : 1);
}

template <int D>
int launch_group_k_pass(const uint8_t *f8, const uint8_t *m4, const uint8_t *l4, const uint8_t *kcm,
                        const unsigned short *q, const unsigned short *k_new, unsigned short *scores,
                        uint8_t *levels_out, const StepGeom &geo, int B, int n_blocks, bool ref, float scale,
                        hipStream_t st, PassShape *shape_only) {
    const int GH = group_heads(geo.G);
    // a wave's set-up (q, levels and masks of GH heads) costs about half a block: several blocks per wave
    int bpw = 1;
    while (bpw < 8 && (int64_t)B * geo.Hkv * (geo.G / GH) * ((n_blocks + 8 * bpw - 1) / (8 * bpw)) * 4 >= 6144) bpw *= 2;
    dim3 grid((n_blocks + 4 * bpw - 1) / (4 * bpw), geo.Hkv * (geo.G / GH), B);
    if (shape_only != nullptr) {
        *shape_only = PassShape{(int)grid.x, (int)grid.y, 4 * bpw * 64};
        return AKV_OK;
    }
#define AKV_GK(RF, GG)                                                                                              \
    hipLaunchKernelGGL((group_k_pass_kernel<D, RF, GG>), grid, dim3(256), 0, st, f8, m4, l4, kcm, q, k_new, scores, \
                       levels_out, geo, bpw, scale)
    if (GH == 4) { if (ref) AKV_GK(true, 4); else AKV_GK(false, 4); }
    else { if (ref) AKV_GK(true, 2); else AKV_GK(false, 2); }
#undef AKV_GK
    return check_launch("decode_step(group k_pass)");
}

template <int D>
int launch_group_v_pass(const uint8_t *f8, const uint8_t *m4, const uint8_t *l4, const unsigned short *probs,
                        const uint8_t *amin, float *partial, uint8_t *levels_out, int levels_stride, uint8_t *amin_out,
                        const StepGeom &geo, int B, const VPlan &p, bool ref, hipStream_t st) {
    const int GH = group_heads(geo.G);
    dim3 grid(p.n_chunks, geo.Hkv * (geo.G / GH), B);
#define AKV_GV(RF, GG)                                                                                                \
    hipLaunchKernelGGL((group_v_pass_kernel<D, RF, GG>), grid, dim3(256), 0, st, f8, m4, l4, probs, amin, partial,    \
                       levels_out, levels_stride, amin_out, geo, p.tokens_per_wave, p.n_chunks)
    if (GH == 4) { if (ref) AKV_GV(true, 4); else AKV_GV(false, 4); }
    else { if (ref) AKV_GV(true, 2); else AKV_GV(false, 2); }
#undef AKV_GV
    return check_launch("decode_step(group v_pass)");
}

#define AKV_INST(DD)                                                                                                     \
    template int launch_group_k_pass<DD>(const uint8_t *, const uint8_t *, const uint8_t *, const uint8_t *,             \
                                         const unsigned short *, const unsigned short *, unsigned short *, uint8_t *,    \
                                         const StepGeom &, int, int, bool, float, hipStream_t, PassShape *);                          \
    template int launch_group_v_pass<DD>(const uint8_t *, const uint8_t *, const uint8_t *, const unsigned short *,      \
                                         const uint8_t *, float *, uint8_t *, int, uint8_t *, const StepGeom &, int,     \
                                         const VPlan &, bool, hipStream_t);
AKV_INST(64)
AKV_INST(128)
AKV_INST(256)
#undef AKV_INST

}  // namespace akv
