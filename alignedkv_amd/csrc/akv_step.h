// Shape and per-sequence state of the fused decode step, shared by its kernels.
#pragma once

#include "akv_cores.h"

namespace akv {

__device__ __forceinline__ u32 exp_field(u32 half_bits) { return (half_bits >> 10) & 0x1fu; }

// Shape and per-sequence state of one step.  Query head hq reads the planes of KV head hq / G (grouped-query
// attention; G == 1 is the reference's multi-head case).  seq_lens (device, may be null) holds the tokens
// cached before this step per sequence; without it every sequence has cur_len tokens.
struct StepGeom {
    int Hq, Hkv, G;
    int cb, max_seq_len, n_max_blocks, row_stride;   // cb: tokens per flush; n_max_blocks: K plane blocks of kb tokens
    int kb;                                          // tokens per K plane block (64 or 256)
    int cur_len;
    int scores_through;    // K pass on 256-token blocks: scores are written through to memory (see k_pass256_split_block)
    const int *seq_lens;
    // per-sequence lengths: workgroup -> {(chunk, head index, batch) of this launch, the sequence's length}, or null
    const u32x2 *task_map;
};

// Launch shape of a pass: grid (grid_x, grid_y, batch), a workgroup covers tokens_per_wg tokens of one sequence.
struct PassShape {
    int grid_x, grid_y, tokens_per_wg;
};
constexpr u32 kNoTask = 0xffffffffu;
__host__ __device__ inline u32 pack_task(int x, int y, int z) { return (u32)x | ((u32)y << 12) | ((u32)z << 20); }
inline bool task_map_fits(const PassShape &s, int B) { return s.grid_x <= 4096 && s.grid_y <= 256 && B <= 4096; }

// tokens flushed into the planes / held in the rest buffer once this step's token has been appended.  The fused step
// flushes 64 tokens at a time (g.cb == 64, checked by the entry points).  UNIFORM: the caller knows that there are no
// per-sequence lengths (no pointer test and no dependent load in front of a one-shot kernel's first requests).
constexpr int kFlush = 64;
template <bool UNIFORM = false>
__device__ __forceinline__ void seq_state(const StepGeom &g, int b, int &R, int &nrest) {
    const int L = ((!UNIFORM && g.seq_lens != nullptr) ? g.seq_lens[b] : g.cur_len) + 1;
    R = L & ~(kFlush - 1);
    nrest = L & (kFlush - 1);
}

// Workgroup -> (chunk x, head index y, batch z) of a launch with grid (chunks, heads, batch); false: nothing to do.
// With per-sequence lengths the grid covers the longest sequence, and in dispatch order (x fastest) the workgroups
// past the end of the shorter ones would be scattered between the working ones, each holding a workgroup slot for
// a microsecond or two (measured: +22 % on the K pass with two such out of three).  The step's first kernel
// therefore writes a map from the linear workgroup index to the tasks that exist, in the same order; what is left
// over gathers at the end of the launch and leaves at once.  An entry also carries the length of its sequence, which
// replaces the look-up in g (the kernel's own copy): one dependent read less in front of a workgroup's first requests.
__device__ __forceinline__ bool step_block(StepGeom &g, int &x, int &y, int &z) {
    x = blockIdx.x;
    y = blockIdx.y;
    z = blockIdx.z;
    if (g.task_map != nullptr) {
        const u32x2 e = g.task_map[blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z)];
        if (e.x == kNoTask) return false;
        x = (int)(e.x & 0xfffu);
        y = (int)((e.x >> 12) & 0xffu);
        z = (int)(e.x >> 20);
        g.cur_len = (int)e.y;
        g.seq_lens = nullptr;
    }
    return true;
}

// Workgroup -> (chunk, query head of the group).  Workgroups go to the 8 XCDs round-robin by linear index,
// and each XCD has its own L2: the G workgroups that stream the same plane chunk for the G query heads of a
// KV head get linear indices 8 apart, i.e. the same XCD at about the same time, so the chunk comes from HBM
// once and from that L2 G-1 times.  gridDim.x = 8 * ceil(chunks / 8) * G.
__device__ __forceinline__ void decode_group_block(int G, int lin, int &chunk, int &gq) {
    if (G == 1) {
        chunk = lin;
        gq = 0;
    } else {
        const int t = lin >> 3;
        gq = t % G;
        chunk = (t / G) * 8 + (lin & 7);
    }
}
static inline int group_grid_x(int chunks, int G) { return G == 1 ? chunks : ((chunks + 7) / 8) * 8 * G; }


// Grouped-query passes (akv_gqa.hip): one workgroup serves group_heads(G) query heads of a KV head.
int group_heads(int G);
template <int D>
int launch_group_k_pass(const uint8_t *f8, const uint8_t *m4, const uint8_t *l4, const uint8_t *kcm,
                        const unsigned short *q, const unsigned short *k_new, unsigned short *scores,
                        uint8_t *levels_out, const StepGeom &geo, int B, int n_blocks, bool ref, float scale,
                        hipStream_t st, PassShape *shape_only = nullptr);
template <int D>
int launch_group_v_pass(const uint8_t *f8, const uint8_t *m4, const uint8_t *l4, const unsigned short *probs,
                        const uint8_t *amin, float *partial, uint8_t *levels_out, int levels_stride, uint8_t *amin_out,
                        const StepGeom &geo, int B, const VPlan &p, bool ref, hipStream_t st);


// Grouped-query passes on the matrix cores (akv_gqa_mfma.hip): 2 to 16 query heads per KV head.
template <int D>
int launch_mfma_k_pass(const uint8_t *f8, const uint8_t *m4, const uint8_t *l4, const uint8_t *kcm,
                       const unsigned short *q, const unsigned short *k_new, unsigned short *scores,
                       uint8_t *levels_out, u32 *prep, const StepGeom &geo, int B, int n_blocks, bool ref, float scale,
                       hipStream_t st, PassShape *shape_only = nullptr, bool prepared = false);
template <int D>
VPlan mfma_v_plan(int B, int Hkv, int n_tokens);
template <int D>
int launch_mfma_v_pass(const uint8_t *f8, const uint8_t *m4, const uint8_t *l4, const unsigned short *probs,
                       const uint8_t *amin, float *partial, uint8_t *levels_out, int levels_stride, uint8_t *amin_out,
                       const StepGeom &geo, int B, const VPlan &p, bool ref, hipStream_t st);
// words of set-up data per (batch, KV head) that launch_mfma_k_pass needs in `prep`
inline size_t mfma_k_prep_words(int D) { return (size_t)64 * (2 * (D / 16) + 4); }

// Set-up of the matrix-core K pass for (batch, KV head) bh_kv, by one wave: lane (j, kq) = (l % 16, l / 16) takes query
// head j of the group at the channels 16 kg + 4 r + kq and leaves, for the K-pass lane of the same index, 2 KG words
// of q (packed fp16 pairs r = 0,1 / 2,3 per channel group) and 4 words of level bits (bit 4 kg + r): this head's
// level is 1 / is 2, and -- OR-ed over the heads of the group -- the mid / last plane row of the channel is fetched.
// kcm may or may not hold this step's token yet: its exponent is folded in here either way.
template <int D, bool REF>
__device__ __forceinline__ void mfma_k_prepare(const uint8_t *__restrict__ kcm, const unsigned short *__restrict__ q,
                                               const unsigned short *__restrict__ k_new, u32 *__restrict__ prep,
                                               uint8_t *__restrict__ levels_out, const StepGeom &geo, int bh_kv) {
    constexpr int KG = D / 16;
    static_assert(4 * KG <= 32, "the level masks are 32 bits wide");
    const int lane = threadIdx.x & 63;
    const int b = bh_kv / geo.Hkv, hkv = bh_kv - b * geo.Hkv;
    const int G = geo.G;
    const int64_t bh0 = (int64_t)b * geo.Hq + hkv * G;
    const int j = lane & 15, kq = lane >> 4;
    const bool head = j < G;
    u32 *out = prep + ((int64_t)bh_kv * 64 + lane) * (2 * KG + 4);
    u32 lv1 = 0, lv2 = 0;
    u32 esum[KG][4];
    u32 mx = 0;
    // Every load first, 16 channels per 16-byte vector (a lane picks its four of them afterwards), none under a
    // branch: a lane without a head reads q out of range and gets zeros.  One round trip instead of one per group.
    const __amdgpu_buffer_rsrc_t rQ = make_rsrc(q + bh0 * D, (u32)(G * D * 2));
    const __amdgpu_buffer_rsrc_t rC = make_rsrc(kcm + (int64_t)bh_kv * D, D);
    const __amdgpu_buffer_rsrc_t rN = make_rsrc(k_new + (int64_t)bh_kv * D, D * 2);
    u32x4 cw[KG], qw[KG][2], nw[KG][2];
#pragma unroll
    for (int kg = 0; kg < KG; ++kg) {
        cw[kg] = __builtin_amdgcn_raw_buffer_load_b128(rC, 16 * kg, 0, 0);
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
            nw[kg][h2] = __builtin_amdgcn_raw_buffer_load_b128(rN, (16 * kg + 8 * h2) * 2, 0, 0);
            qw[kg][h2] = __builtin_amdgcn_raw_buffer_load_b128(rQ, head ? (j * D + 16 * kg + 8 * h2) * 2 : kSkip, 0, 0);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    // channel 16 kg + 4 r + kq: byte kq of word r of the column maxima, half (kq & 1) of word 2 (r & 1) + kq / 2 of
    // vector r / 2 of q and the new key
    auto half_at = [&](const u32x4 (&v)[2], int r) -> u32 {
        const u32x4 w = v[r >> 1];
        const u32 lo = (r & 1) ? w.z : w.x, hi = (r & 1) ? w.w : w.y;
        const u32 word = (kq & 2) ? hi : lo;
        return (kq & 1) ? word >> 16 : word & 0xffffu;
    };
#pragma unroll
    for (int kg = 0; kg < KG; ++kg) {
        u32 qb[4];
        const u32 cws[4] = {cw[kg].x, cw[kg].y, cw[kg].z, cw[kg].w};
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            qb[r] = half_at(qw[kg], r);
            // column max including the token appended by this step
            const u32 cm = max((cws[r] >> (8 * kq)) & 0xffu, exp_field(half_at(nw[kg], r)));
            esum[kg][r] = (exp_field(qb[r]) + cm) & 0xffu;
            mx = max(mx, esum[kg][r]);
        }
        out[2 * kg] = qb[0] | (qb[1] << 16);
        out[2 * kg + 1] = qb[2] | (qb[3] << 16);
    }
    mx = max(mx, (u32)__shfl_xor((int)mx, 16, 64));
    mx = max(mx, (u32)__shfl_xor((int)mx, 32, 64));
#pragma unroll
    for (int kg = 0; kg < KG; ++kg)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int lv = REF ? 0 : k_level((unsigned char)mx, (unsigned char)esum[kg][r]);
            if (head) {
                lv1 |= (lv == 1 ? 1u : 0u) << (4 * kg + r);
                lv2 |= (lv == 2 ? 1u : 0u) << (4 * kg + r);
                if (levels_out != nullptr) levels_out[(bh0 + j) * D + 16 * kg + 4 * r + kq] = (uint8_t)lv;
            }
        }
    // a plane row is fetched if any head of the group reads it: OR over the 16 lanes that share kq
    u32 need_mid = head ? ~lv2 : 0u;
    u32 need_last = head ? ~(lv1 | lv2) : 0u;
#pragma unroll
    for (int m = 1; m < 16; m <<= 1) {
        need_mid |= (u32)__shfl_xor((int)need_mid, m, 64);
        need_last |= (u32)__shfl_xor((int)need_last, m, 64);
    }
    out[2 * KG] = lv1;
    out[2 * KG + 1] = lv2;
    out[2 * KG + 2] = need_mid;
    out[2 * KG + 3] = need_last;
}

}  // namespace akv
