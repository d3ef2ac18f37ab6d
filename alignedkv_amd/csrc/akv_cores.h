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
    // Partners 32 and 16 lanes apart exchange through the half-wave / row swap instructions (one instruction per
    // pair of sums, no LDS round trip); the sums are the same bits as with a shuffle (own + partner's either way).
    if (lane_mask == 32 || lane_mask == 16) {
#pragma unroll
        for (int i = 0; i < N / 2; ++i) {
            const u32 x = __float_as_uint(a[i]), y = __float_as_uint(a[i + N / 2]);
            if (lane_mask == 32) {
                const auto r = __builtin_amdgcn_permlane32_swap(x, y, false, false);
                a[i] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
            } else {
                const auto r = __builtin_amdgcn_permlane16_swap(x, y, false, false);
                a[i] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
            }
        }
        return;
    }
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
template <int HG>
struct KHalfTile {   // HG load groups of one block: 16 channels x 64 slots each
    u32x4 h[HG];
    u32x2 m[HG], l[HG];
};

template <int D, int HG>
__device__ __forceinline__ void k_issue_half_h(KHalfTile<HG> &t, const __amdgpu_buffer_rsrc_t rH, int blk, int g0) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int g = 0; g < HG; ++g)
        t.h[g] = __builtin_amdgcn_raw_buffer_load_b128(rH, blk * (D * 64) + (g0 + g) * 1024 + lane * 16, 00, kStream);
}

template <int D, int HG>
__device__ __forceinline__ void k_issue_half_ml(KHalfTile<HG> &t, const __amdgpu_buffer_rsrc_t rM,
                                                const __amdgpu_buffer_rsrc_t rL, int blk, int g0, u32 need_mid,
                                                u32 need_last) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int g = 0; g < HG; ++g) {
        const int gg = g0 + g;
        const int mo = ((need_mid >> gg) & 1u) ? blk * (D * 32) + gg * 512 + lane * 8 : kSkip;
        const int lo = ((need_last >> gg) & 1u) ? blk * (D * 32) + gg * 512 + lane * 8 : kSkip;
        t.m[g] = __builtin_amdgcn_raw_buffer_load_b64(rM, mo, 00, kStream);
        t.l[g] = __builtin_amdgcn_raw_buffer_load_b64(rL, lo, 00, kStream);
    }
}

template <int D, int HG>
__device__ __forceinline__ void k_issue_half(KHalfTile<HG> &t, const __amdgpu_buffer_rsrc_t rH,
                                             const __amdgpu_buffer_rsrc_t rM, const __amdgpu_buffer_rsrc_t rL, int blk,
                                             int g0, u32 need_mid, u32 need_last) {
    k_issue_half_h<D, HG>(t, rH, blk, g0);
    k_issue_half_ml<D, HG>(t, rM, rL, blk, g0, need_mid, need_last);
}

// The high-byte rows of the wave's first half tile do not depend on the fetch levels: a kernel calls this
// first, works out q and the levels while the loads are in flight, then calls k_score_blocks.
template <int D>
__device__ __forceinline__ void k_prefetch_first(KHalfTile<D / 32> &ta, const uint8_t *f8, int n_blocks, int first_blk) {
    k_issue_half_h<D, D / 32>(ta, make_rsrc(f8, (u32)n_blocks * (D * 64)), first_blk, 0);
    __builtin_amdgcn_sched_barrier(0);
}

template <int HG>
__device__ __forceinline__ void k_compute_half(float *acc, const KHalfTile<HG> &t, int g0, const float *qf,
                                               u32 need_mid, u32 need_last) {
#pragma unroll
    for (int g = 0; g < HG; ++g) {
        const int gg = g0 + g;
        const u32 cm = ((need_mid >> gg) & 1u) ? 0u : 0x88888888u;                                 // level 2
        const u32 cl = (((need_mid >> gg) & 1u) && !((need_last >> gg) & 1u)) ? 0x88888888u : 0u;  // level 1
        fma8(acc, t.h[g].x, t.h[g].y, t.m[g].x | cm, t.l[g].x | cl, qf[gg]);
        fma8(acc + 8, t.h[g].z, t.h[g].w, t.m[g].y | cm, t.l[g].y | cl, qf[gg]);
    }
}

// Software pipeline over half blocks: while one half tile is being multiplied, the loads of the next
// half tile (same block or the wave's next block) are in flight.
template <int D>
__device__ __forceinline__ void k_score_blocks(KHalfTile<D / 32> &ta, const uint8_t *f8, const uint8_t *m4,
                                               const uint8_t *l4, int n_blocks, int first_blk, int end_blk,
                                               const float *qf, u32 need_mid, u32 need_last, unsigned short *s_row,
                                               float scale, int blk_stride = 1, bool through = true) {
    constexpr int CB = 64;
    constexpr int NG = D / 16;
    constexpr int HG = NG / 2;
    const int lane = threadIdx.x & 63;
    const __amdgpu_buffer_rsrc_t rH = make_rsrc(f8, (u32)n_blocks * (D * CB));
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(m4, (u32)n_blocks * (D * CB / 2));
    const __amdgpu_buffer_rsrc_t rL = make_rsrc(l4, (u32)n_blocks * (D * CB / 2));
    const __amdgpu_buffer_rsrc_t rS = make_rsrc(s_row, (u32)n_blocks * CB * 2);
    const int slot = (lane & 3) * 16 + ((lane & 32) ? 8 : 0) + ((lane & 16) ? 4 : 0) + ((lane & 8) ? 2 : 0) +
                     ((lane & 4) ? 1 : 0);
    // sched_barrier(0): the instruction scheduler must not move loads or arithmetic across the phase
    // boundaries, otherwise it merges the two half tiles into one wait-for-everything block.  Every wait
    // in the loop sees exactly one younger half tile in flight, from the prologue and from the back edge.
    KHalfTile<HG> tb;
    k_issue_half_ml<D, HG>(ta, rM, rL, first_blk, 0, need_mid, need_last);   // its high bytes: k_prefetch_first
    __builtin_amdgcn_sched_barrier(0);
    for (int blk = first_blk; blk < end_blk; blk += blk_stride) {
        float acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
        k_issue_half<D, HG>(tb, rH, rM, rL, blk, HG, need_mid, need_last);
        __builtin_amdgcn_sched_barrier(0);
        k_compute_half<HG>(acc, ta, 0, qf, need_mid, need_last);
        __builtin_amdgcn_sched_barrier(0);
        // past the last block the offsets fall outside the buffer resources: the loads return 0 and fetch nothing
        k_issue_half<D, HG>(ta, rH, rM, rL, blk + blk_stride < end_blk ? blk + blk_stride : n_blocks, 0, need_mid, need_last);
        __builtin_amdgcn_sched_barrier(0);
        k_compute_half<HG>(acc, tb, HG, qf, need_mid, need_last);
        __builtin_amdgcn_sched_barrier(0);
        // acc[i]: partial score of slot (lane&3)*16 + i over this lane's channels
        reduce_scatter_step<16>(acc, 32);
        reduce_scatter_step<8>(acc, 16);
        reduce_scatter_step<4>(acc, 8);
        reduce_scatter_step<2>(acc, 4);
        store_score(rS, (blk * CB + slot) * 2, float_to_half_bits(acc[0] * scale), through);
    }
}

// One block with everything in flight at once: the caller has requested the high bytes of all its channels
// (k_issue_half_h<D, D / 16>) before working out q and the levels; here the nibble rows follow, then the arithmetic.
// 16 KiB per wave and no loop: for kernels that give every block a wave of its own.
template <int D>
__device__ __forceinline__ void k_score_block_whole(KHalfTile<D / 16> &t, const uint8_t *m4, const uint8_t *l4, int n_blocks,
                                                    int blk, const float *qf, u32 need_mid, u32 need_last,
                                                    unsigned short *s_row, float scale, bool through = true) {
    constexpr int CB = 64;
    constexpr int NG = D / 16;
    const int lane = threadIdx.x & 63;
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(m4, (u32)n_blocks * (D * CB / 2));
    const __amdgpu_buffer_rsrc_t rL = make_rsrc(l4, (u32)n_blocks * (D * CB / 2));
    const __amdgpu_buffer_rsrc_t rS = make_rsrc(s_row, (u32)n_blocks * CB * 2);
    const int slot = (lane & 3) * 16 + ((lane & 32) ? 8 : 0) + ((lane & 16) ? 4 : 0) + ((lane & 8) ? 2 : 0) +
                     ((lane & 4) ? 1 : 0);
    k_issue_half_ml<D, NG>(t, rM, rL, blk, 0, need_mid, need_last);
    __builtin_amdgcn_sched_barrier(0);
    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    k_compute_half<NG>(acc, t, 0, qf, need_mid, need_last);
    reduce_scatter_step<16>(acc, 32);
    reduce_scatter_step<8>(acc, 16);
    reduce_scatter_step<4>(acc, 8);
    reduce_scatter_step<2>(acc, 4);
    store_score(rS, (blk * CB + slot) * 2, float_to_half_bits(acc[0] * scale), through);
}

// ------------------------------------------------------------------------------------------------
// V: one wave accumulates tokens [t_begin, t_end) of one (batch, head) into acc[16].
//   f8/m4/l4 point at token 0 of this (batch, head); n_tokens bounds the buffer resources.
//   Lane layout: lane -> token (lane / (D/16)) of each wave-wide load, channels (lane % (D/16))*16..+16.
//   s_row: fp16 probabilities of this (batch, head).  levels_row (may be null): level per token.
// ------------------------------------------------------------------------------------------------
// Empty volatile asm that reads and writes the 16 accumulators: pins the arithmetic that produced them
// before this point and everything after it behind (the compiler otherwise sinks side-effect-free
// multiply-adds past later loads and branches, which undoes the software pipeline).
__device__ __forceinline__ void pin_accumulators(float *a) {
    asm volatile("" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]),
                      "+v"(a[8]), "+v"(a[9]), "+v"(a[10]), "+v"(a[11]), "+v"(a[12]), "+v"(a[13]), "+v"(a[14]), "+v"(a[15]));
}

// ------------------------------------------------------------------------------------------------
// K with 256-token plane blocks (d_block == 256): scores of blocks [first_blk, end_blk) of one (batch, head).
// A channel's row of a block is 256 B of high bytes and 128 B in each nibble plane, so a skipped nibble row is
// a whole 128-byte line: HBM delivers exactly the bytes the levels ask for (with 64-token blocks a 32-byte row
// shares its line with three other channels).
//   Lane layout: lane -> channel 4 g + lane/16 of load group g (4 channels), slots (lane & 15) * 16 .. + 16.
//   bit g of need_mid / need_last: fetch that plane row of the lane's channel in group g.
//   valid_tokens: scores of tokens at and beyond it are not stored (the last block may be partly filled).
// The 4 lanes of a slot range hold 16 partial sums each: two reduce-scatter steps (12 shuffles per 256 tokens,
// against 15 per 64 tokens in the 64-token layout) leave 4 consecutive scores per lane.
// ------------------------------------------------------------------------------------------------
template <int D, int HG>
__device__ __forceinline__ void k256_issue_h(KHalfTile<HG> &t, const __amdgpu_buffer_rsrc_t rH, int blk, int g0) {
    const int lane = threadIdx.x & 63;
    const int cs = lane >> 4, piece = lane & 15;
#pragma unroll
    for (int g = 0; g < HG; ++g) {
        const int c = 4 * (g0 + g) + cs;
        t.h[g] = __builtin_amdgcn_raw_buffer_load_b128(rH, blk * (D * 256) + c * 256 + piece * 16, 00, kStream);
    }
}

template <int D, int HG>
__device__ __forceinline__ void k256_issue_ml(KHalfTile<HG> &t, const __amdgpu_buffer_rsrc_t rM, const __amdgpu_buffer_rsrc_t rL,
                                              int blk, int g0, u32 need_mid, u32 need_last) {
    const int lane = threadIdx.x & 63;
    const int cs = lane >> 4, piece = lane & 15;
#pragma unroll
    for (int g = 0; g < HG; ++g) {
        const int gg = g0 + g, c = 4 * gg + cs;
        const int off = blk * (D * 128) + c * 128 + piece * 8;
        t.m[g] = __builtin_amdgcn_raw_buffer_load_b64(rM, ((need_mid >> gg) & 1u) ? off : kSkip, 00, kStream);
        t.l[g] = __builtin_amdgcn_raw_buffer_load_b64(rL, ((need_last >> gg) & 1u) ? off : kSkip, 00, kStream);
    }
}

template <int D, int HG>
__device__ __forceinline__ void k256_issue(KHalfTile<HG> &t, const __amdgpu_buffer_rsrc_t rH, const __amdgpu_buffer_rsrc_t rM,
                                           const __amdgpu_buffer_rsrc_t rL, int blk, int g0, u32 need_mid, u32 need_last) {
    k256_issue_h<D, HG>(t, rH, blk, g0);
    k256_issue_ml<D, HG>(t, rM, rL, blk, g0, need_mid, need_last);
}

// The high-byte rows of the wave's first half tile do not depend on the fetch levels: a kernel calls this first,
// works out q and the levels while the loads are in flight, then calls k256_score_blocks.
template <int D>
__device__ __forceinline__ void k256_prefetch_first(KHalfTile<4> &ta, const uint8_t *f8, int n_blocks, int first_blk) {
    k256_issue_h<D, 4>(ta, make_rsrc(f8, (u32)n_blocks * (D * 256)), first_blk, 0);
    __builtin_amdgcn_sched_barrier(0);
}

template <int D>
__device__ __forceinline__ void k256_score_blocks(KHalfTile<4> &ta, const uint8_t *f8, const uint8_t *m4, const uint8_t *l4, int n_blocks,
                                                  int first_blk, int end_blk, u32 *qh, u32 need_mid, u32 need_last,
                                                  unsigned short *s_row, int valid_tokens, float scale) {
    // qh[g / 2]: q of the lane's channels of groups g (low half) and g + 1 (high half), fp16
    constexpr int CB = 256;
    constexpr int NG = D / 4;      // load groups of 4 channels
    constexpr int HG = 4;          // groups per half tile: 8 KiB per wave in flight
    static_assert(NG % (2 * HG) == 0 && NG <= 32, "head_dim 64 or 128");
    const int lane = threadIdx.x & 63;
    const __amdgpu_buffer_rsrc_t rH = make_rsrc(f8, (u32)n_blocks * (D * CB));
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(m4, (u32)n_blocks * (D * CB / 2));
    const __amdgpu_buffer_rsrc_t rL = make_rsrc(l4, (u32)n_blocks * (D * CB / 2));
    const __amdgpu_buffer_rsrc_t rS = make_rsrc(s_row, (u32)valid_tokens * 2);
    const int slot = (lane & 15) * 16 + ((lane & 32) ? 8 : 0) + ((lane & 16) ? 4 : 0);
    KHalfTile<HG> tb;
    k256_issue_ml<D, HG>(ta, rM, rL, first_blk, 0, need_mid, need_last);   // its high bytes: k256_prefetch_first
    __builtin_amdgcn_sched_barrier(0);
    for (int blk = first_blk; blk < end_blk; ++blk) {
        float acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
        // the substitution bytes derived from these masks are cheap to rebuild; kept across the loop they would
        // take 64 registers: hide their loop invariance from the compiler
        asm volatile("" : "+v"(need_mid), "+v"(need_last));
#pragma unroll
        for (int g0 = 0; g0 < NG; g0 += 2 * HG) {
            // q stays packed in registers (16 instead of 32): unpack the 8 values of this pair of half tiles
            float qf[NG];
#pragma unroll
            for (int g = g0; g < g0 + 2 * HG; g += 2) {
                u32 w = qh[g >> 1];
                asm volatile("" : "+v"(w));
                qf[g] = lo_half_to_float(w);
                qf[g + 1] = hi_half_to_float(w);
            }
            k256_issue<D, HG>(tb, rH, rM, rL, blk, g0 + HG, need_mid, need_last);
            __builtin_amdgcn_sched_barrier(0);
            k_compute_half<HG>(acc, ta, g0, qf, need_mid, need_last);
            pin_accumulators(acc);
            __builtin_amdgcn_sched_barrier(0);
            // past the last block the offsets fall outside the buffer resources: nothing is fetched
            if (g0 + 2 * HG < NG) k256_issue<D, HG>(ta, rH, rM, rL, blk, g0 + 2 * HG, need_mid, need_last);
            else k256_issue<D, HG>(ta, rH, rM, rL, blk + 1 < end_blk ? blk + 1 : n_blocks, 0, need_mid, need_last);
            __builtin_amdgcn_sched_barrier(0);
            k_compute_half<HG>(acc, tb, g0 + HG, qf, need_mid, need_last);
            pin_accumulators(acc);
            __builtin_amdgcn_sched_barrier(0);
        }
        reduce_scatter_step<16>(acc, 32);
        reduce_scatter_step<8>(acc, 16);
        const u32 w0 = (u32)float_to_half_bits(acc[0] * scale) | ((u32)float_to_half_bits(acc[1] * scale) << 16);
        const u32 w1 = (u32)float_to_half_bits(acc[2] * scale) | ((u32)float_to_half_bits(acc[3] * scale) << 16);
        // device scope: the workgroup that runs the softmax for this (batch, head) may sit on another XCD
        __builtin_amdgcn_raw_buffer_store_b64((u32x2){w0, w1}, rS, (blk * CB + slot) * 2, 0, kDeviceScope);
    }
}

template <int HV>
struct VHighPart {   // HV wave-wide loads: 64/(D/16) token rows each, high bytes
    u32x4 h[HV];
};
template <int HV>
struct VLowPart {    // the nibble rows of the same tokens
    u32x2 m[HV], l[HV];
    u32 cm[HV], cl[HV];   // substitution bytes of skipped planes
};
template <int HV>
struct VHalfTile : VHighPart<HV>, VLowPart<HV> {};

// Requests the rows of the tokens base + u*TPL + tl (u < HV).  The high-byte rows do not depend on the
// fetch level and are requested before the probabilities (sb) are looked at.
template <int D, int HV>
__device__ __forceinline__ void v_issue_half_h(VHighPart<HV> &t, const __amdgpu_buffer_rsrc_t rH, int base, int t_end) {
    constexpr int LPR = D / 16, TPL = 64 / LPR;
    const int lane = threadIdx.x & 63;
    const int tl = lane / LPR, cl = lane % LPR;
#pragma unroll
    for (int u = 0; u < HV; ++u) {
        const int tok = base + u * TPL + tl;
        t.h[u] = __builtin_amdgcn_raw_buffer_load_b128(rH, tok < t_end ? tok * D + cl * 16 : kSkip, 0, kStream);
    }
}

template <int D, bool REF, int HV>
__device__ __forceinline__ void v_issue_half_ml(VLowPart<HV> &t, const __amdgpu_buffer_rsrc_t rM,
                                                const __amdgpu_buffer_rsrc_t rL, int base, int t_end, const u32 *sb,
                                                unsigned char amin) {
    constexpr int LPR = D / 16, TPL = 64 / LPR;
    const int lane = threadIdx.x & 63;
    const int tl = lane / LPR, cl = lane % LPR;
#pragma unroll
    for (int u = 0; u < HV; ++u) {
        const int tok = base + u * TPL + tl;
        const bool valid = tok < t_end;
        const int level = REF ? 0 : v_level(amin, (unsigned short)sb[u]);
        t.m[u] = __builtin_amdgcn_raw_buffer_load_b64(rM, (valid && level < 2) ? tok * (D / 2) + cl * 8 : kSkip, 00, kStream);
        t.l[u] = __builtin_amdgcn_raw_buffer_load_b64(rL, (valid && level == 0) ? tok * (D / 2) + cl * 8 : kSkip, 00, kStream);
        t.cm[u] = level == 2 ? 0x88888888u : 0u;
        t.cl[u] = level == 1 ? 0x88888888u : 0u;
    }
}

template <int D>
struct VFirstTile {
    VHalfTile<(D / 16 < 8 ? D / 16 : 8) / 2> t;
};

// The high-byte rows of the wave's first half tile depend on nothing: a kernel calls this first, then loads
// the threshold, then calls v_accumulate.
template <int D>
__device__ __forceinline__ void v_prefetch_first(VFirstTile<D> &ft, const uint8_t *f8, int n_tokens, int t_begin, int t_end) {
    v_issue_half_h<D, (D / 16 < 8 ? D / 16 : 8) / 2>(ft.t, make_rsrc(f8, (u32)n_tokens * D), t_begin, t_end);
    __builtin_amdgcn_sched_barrier(0);
}

template <int HV>
__device__ __forceinline__ void v_compute_half(float *acc, const VHighPart<HV> &th, const VLowPart<HV> &t, const u32 *sb) {
#pragma unroll
    for (int u = 0; u < HV; ++u) {
        const float sf = half_bits_to_float(sb[u]);
        fma8(acc, th.h[u].x, th.h[u].y, t.m[u].x | t.cm[u], t.l[u].x | t.cl[u], sf);
        fma8(acc + 8, th.h[u].z, th.h[u].w, t.m[u].y | t.cm[u], t.l[u].y | t.cl[u], sf);
    }
}
template <int HV>
__device__ __forceinline__ void v_compute_half(float *acc, const VHalfTile<HV> &t, const u32 *sb) {
    v_compute_half<HV>(acc, t, t, sb);
}

// A half tile whose tokens are all at level 2 (wave-uniform): only the high bytes are requested and multiplied,
// the low byte is the constant 0x80.  With ~1 % of the tokens below level 2 that is most half tiles, and it
// saves two thirds of their load instructions (skipped nibble rows still cost an issue slot each).
template <int HV>
__device__ __forceinline__ void v_compute_half_coarse(float *acc, const VHighPart<HV> &t, const u32 *sb) {
#pragma unroll
    for (int u = 0; u < HV; ++u) {
        const float sf = half_bits_to_float(sb[u]);
        fma8_even_odd(acc, t.h[u].x, t.h[u].y, 0x80808080u, 0x80808080u, sf);
        fma8_even_odd(acc + 8, t.h[u].z, t.h[u].w, 0x80808080u, 0x80808080u, sf);
    }
}

template <bool REF, int HV>
__device__ __forceinline__ bool v_half_is_fine(const u32 *sb, unsigned char amin) {
    if (REF) return true;
    bool any = false;
#pragma unroll
    for (int u = 0; u < HV; ++u) any = any || v_level(amin, (unsigned short)sb[u]) < 2;
    return __builtin_amdgcn_ballot_w64(any) != 0ull;
}

// ---- tokens below level 2, taken out of the streaming loops -----------------------------------------
// With ~1 % of the tokens below level 2, 25-80 % of the 32-token half tiles hold one; fetching those half tiles' nibble
// rows inside the pipeline holds a wave up by about 0.7 us each (measured).  The loops therefore multiply every token
// at level 2 (high bytes only); a lane whose token is below level 2 appends (token, probability) to the wave's list in
// LDS, and the wave then adds p * (value at the token's level - value at level 2) for the listed tokens, TPL at a
// time.  Both values are fp16 numbers, so the result differs from multiplying the token at its level only by fp32
// rounding.
template <int D>
struct VListed {
    static constexpr int LPR = D / 16, TPL = 64 / LPR;
    struct Step {
        u32x4 h;
        u32x2 m, l;
        u32 cm, cl;
        float p;
    };
    // Appends the lanes' tokens flagged `fine` (one lane per token: the first of its row) to list[count...].
    static __device__ __forceinline__ void append(u32 *list, int &count, bool fine, int tok, u32 prob_bits) {
        const unsigned long long m = __builtin_amdgcn_ballot_w64(fine);
        if (m == 0ull) return;
        const int before = (int)__builtin_amdgcn_mbcnt_hi((u32)(m >> 32), __builtin_amdgcn_mbcnt_lo((u32)m, 0u));
        if (fine) list[count + before] = (u32)tok | (prob_bits << 16);
        count += __builtin_popcountll(m);
    }
    // lane group tl takes entry e0 + tl; an entry holds its token relative to tok_base in 16 bits
    static __device__ __forceinline__ void request(Step &st, const u32 *list, int count, int e0, const __amdgpu_buffer_rsrc_t rH,
                                                   const __amdgpu_buffer_rsrc_t rM, const __amdgpu_buffer_rsrc_t rL,
                                                   unsigned char amin, int tok_base) {
        const int lane = threadIdx.x & 63, tl = lane / LPR, cl = lane % LPR;
        const int e = e0 + tl;
        const bool on = e < count;
        const u32 entry = on ? list[e] : 0u;
        const int tok = tok_base + (int)(entry & 0xffffu);
        const u32 pb = entry >> 16;
        const int level = v_level(amin, (unsigned short)pb);
        st.h = __builtin_amdgcn_raw_buffer_load_b128(rH, on ? tok * D + cl * 16 : kSkip, 0, kStream);
        st.m = __builtin_amdgcn_raw_buffer_load_b64(rM, (on && level < 2) ? tok * (D / 2) + cl * 8 : kSkip, 0, kStream);
        st.l = __builtin_amdgcn_raw_buffer_load_b64(rL, (on && level == 0) ? tok * (D / 2) + cl * 8 : kSkip, 0, kStream);
        st.cm = level == 2 ? 0x88888888u : 0u;
        st.cl = level == 1 ? 0x88888888u : 0u;
        st.p = on ? half_bits_to_float(pb) : 0.f;
    }
    static __device__ __forceinline__ void apply(float *acc, const Step &st) {
        fma8(acc, st.h.x, st.h.y, st.m.x | st.cm, st.l.x | st.cl, st.p);
        fma8(acc + 8, st.h.z, st.h.w, st.m.y | st.cm, st.l.y | st.cl, st.p);
        fma8_even_odd(acc, st.h.x, st.h.y, 0x80808080u, 0x80808080u, -st.p);
        fma8_even_odd(acc + 8, st.h.z, st.h.w, 0x80808080u, 0x80808080u, -st.p);
    }
    // the list from entry e0 on; `first` holds the entries e0 .. e0 + TPL - 1, requested by the caller earlier
    static __device__ __forceinline__ void apply_all(float *acc, Step &first, const u32 *list, int count,
                                                     const __amdgpu_buffer_rsrc_t rH, const __amdgpu_buffer_rsrc_t rM,
                                                     const __amdgpu_buffer_rsrc_t rL, unsigned char amin, int tok_base,
                                                     int e0 = 0) {
        if (count <= e0) return;
        if (count <= e0 + TPL) {       // the usual case: nothing more to request (and to wait for)
            apply(acc, first);
            return;
        }
        Step other;
        for (; e0 < count; e0 += 2 * TPL) {
            request(other, list, count, e0 + TPL, rH, rM, rL, amin, tok_base);
            __builtin_amdgcn_sched_barrier(0);
            apply(acc, first);
            __builtin_amdgcn_sched_barrier(0);
            request(first, list, count, e0 + 2 * TPL, rH, rM, rL, amin, tok_base);
            __builtin_amdgcn_sched_barrier(0);
            apply(acc, other);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
};

// PAUX: cache policy of the probability loads (kDeviceScope when another workgroup of the same launch wrote them)
// PREFETCHED: the caller has requested the first half tile's high bytes (v_prefetch_first); otherwise they are requested
// here, behind the probabilities -- loads come back in the order they were issued, so the small loads that the fetch
// levels depend on go first where nothing else has to happen in between.
// PROWS: the probabilities of the wave's tokens are requested as one row (8 bytes a lane) and spread through LDS; for
// callers whose rows are 8-byte aligned and whose token ranges are multiples of 4 (the fused step).  Otherwise every lane
// requests its own, two bytes at a time: a wave-wide request then brings 64 / (D / 16) probabilities, 32 requests for
// the 256 tokens of a wave at head_dim 128.
template <int D, bool REF, int NIT, int PAUX = 0, bool PREFETCHED = true, bool PROWS = false>
__device__ __forceinline__ void v_accumulate(VFirstTile<D> &ft, const uint8_t *f8, const uint8_t *m4, const uint8_t *l4,
                                             int n_tokens, const unsigned short *s_row, unsigned char amin, int t_begin,
                                             int t_end, float *acc, uint8_t *levels_row) {
    constexpr int LPR = D / 16;            // lanes per token row
    constexpr int TPL = 64 / LPR;          // token rows per wave-wide load
    constexpr int U = LPR < 8 ? LPR : 8;   // wave-wide loads per batch of 64 (32 for head_dim 256) tokens
    constexpr int HV = U / 2;              // loads per half tile
    constexpr int NH = 2 * NIT;            // half tiles per wave
    const int lane = threadIdx.x & 63;
    const int tl = lane / LPR;
    const __amdgpu_buffer_rsrc_t rH = make_rsrc(f8, (u32)n_tokens * D);
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(m4, (u32)n_tokens * (D / 2));
    const __amdgpu_buffer_rsrc_t rL = make_rsrc(l4, (u32)n_tokens * (D / 2));
    const __amdgpu_buffer_rsrc_t rS = make_rsrc(s_row, (u32)n_tokens * 2);
    // The probabilities of all the wave's tokens first: the fetch level of a token depends on its
    // probability, and a load per batch would put a memory round trip in front of every batch.
    u32 sb[NH][HV];
    if constexpr (PROWS) {
        constexpr int NK = NH * HV, NTOK = NK * TPL;      // loads and tokens per wave
        static_assert(NTOK <= 256 && NK % 2 == 0, "one 8-byte request per lane covers the wave's tokens");
        __shared__ __attribute__((aligned(16))) unsigned short prob_rows[4][TPL * NK];   // per wave: [token row of a load][load]
        unsigned short *wp = prob_rows[threadIdx.x >> 6];
        const int i0 = 4 * lane, t0 = t_begin + i0;
        const u32x2 four = __builtin_amdgcn_raw_buffer_load_b64(rS, (i0 < NTOK && t0 < t_end) ? t0 * 2 : kSkip, 0, PAUX);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (!PREFETCHED) v_prefetch_first<D>(ft, f8, n_tokens, t_begin, t_end);
        __builtin_amdgcn_sched_barrier(0);
        if (i0 < NTOK) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int i = i0 + e;     // token i of the wave: row i % TPL of load i / TPL
                wp[(i % TPL) * NK + i / TPL] = (unsigned short)(((e & 2) ? four.y : four.x) >> (16 * (e & 1)));
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // read by other lanes of the wave
        u32 pw[NK / 2];
#pragma unroll
        for (int w = 0; w < NK / 2; ++w) pw[w] = *reinterpret_cast<const u32 *>(wp + tl * NK + 2 * w);
#pragma unroll
        for (int hf = 0; hf < NH; ++hf)
#pragma unroll
            for (int u = 0; u < HV; ++u) {
                const int k = hf * HV + u;
                sb[hf][u] = (pw[k >> 1] >> (16 * (k & 1))) & 0xffffu;
            }
    } else {
#pragma unroll
    for (int hf = 0; hf < NH; ++hf)
#pragma unroll
        for (int u = 0; u < HV; ++u) {
            const int t = t_begin + (hf * HV + u) * TPL + tl;
            sb[hf][u] = (u32)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(rS, t < t_end ? t * 2 : kSkip, 0, PAUX);
        }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (!PREFETCHED) v_prefetch_first<D>(ft, f8, n_tokens, t_begin, t_end);
    }
    // Software pipeline over half tiles (see k_score_blocks): one half tile is in flight while the other is
    // multiplied; sched_barrier(0) keeps the instruction scheduler from merging the phases.
    VHalfTile<HV> &ta = ft.t;
    VHalfTile<HV> tb;
    bool fine[NH];   // wave-uniform: some token of the half tile is below level 2
#pragma unroll
    for (int hf = 0; hf < NH; ++hf) fine[hf] = v_half_is_fine<REF, HV>(sb[hf], amin);
    if (fine[0]) v_issue_half_ml<D, REF, HV>(ta, rM, rL, t_begin, t_end, sb[0], amin);   // its high bytes: v_prefetch_first
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int hf = 0; hf < NH; hf += 2) {
        v_issue_half_h<D, HV>(tb, rH, t_begin + (hf + 1) * HV * TPL, t_end);
        if (fine[hf + 1]) v_issue_half_ml<D, REF, HV>(tb, rM, rL, t_begin + (hf + 1) * HV * TPL, t_end, sb[hf + 1], amin);
        __builtin_amdgcn_sched_barrier(0);
        if (fine[hf]) v_compute_half<HV>(acc, ta, sb[hf]);
        else v_compute_half_coarse<HV>(acc, ta, sb[hf]);
        pin_accumulators(acc);
        __builtin_amdgcn_sched_barrier(0);
        if (hf + 2 < NH) {
            v_issue_half_h<D, HV>(ta, rH, t_begin + (hf + 2) * HV * TPL, t_end);
            if (fine[hf + 2]) v_issue_half_ml<D, REF, HV>(ta, rM, rL, t_begin + (hf + 2) * HV * TPL, t_end, sb[hf + 2], amin);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (fine[hf + 1]) v_compute_half<HV>(acc, tb, sb[hf + 1]);
        else v_compute_half_coarse<HV>(acc, tb, sb[hf + 1]);
        pin_accumulators(acc);
        __builtin_amdgcn_sched_barrier(0);
    }
    // optional record of the levels, outside the pipeline (a store under a branch inside it would split
    // the loop body into blocks and let the compiler sink the arithmetic past the loads)
    if (levels_row != nullptr && (lane % LPR) == 0) {
#pragma unroll
        for (int hf = 0; hf < NH; ++hf)
#pragma unroll
            for (int u = 0; u < HV; ++u) {
                const int t = t_begin + (hf * HV + u) * TPL + tl;
                if (t < t_end) levels_row[t] = (uint8_t)(REF ? 0 : v_level(amin, (unsigned short)sb[hf][u]));
            }
    }
}

// One wave streams its share of the half tiles of a row of V planes (VSeq; a half tile = HT tokens): a ring of NR half tiles of high bytes, each requested together with its probabilities NR - 1 half tiles
// before it is multiplied (neither depends on a fetch level); the nibble rows of a half tile with a token below
// level 2 are requested one half tile ahead, before the newest high bytes, so that waiting for them does not wait
// for those.  For callers that give a wave a long range: v_accumulate keeps one half tile in flight and leaves the
// overlap to the number of waves.
template <int D>
struct VStream {
    static constexpr int LPR = D / 16, TPL = 64 / LPR, U = LPR < 8 ? LPR : 8, HV = U / 2, HT = HV * TPL;
};

template <int D, int NR>
struct VRing {
    VHighPart<VStream<D>::HV> hi[NR];
    u32 sb[NR][VStream<D>::HV];
};

// A wave's share of the half tiles of a row: its i-th half tile is start + i * stride (i < count), so that at any time
// the waves of a workgroup read neighbouring rows.  Past the share: n_halves (nothing is fetched).
struct VSeq {
    int start, stride, count, n_halves;
    __device__ __forceinline__ int half(int i) const { return i < count ? start + i * stride : n_halves; }
    __device__ __forceinline__ int left() const { return count; }
};

// High bytes of half tile `half`: one address per lane, the HV rows at constant distances from it.  A half tile past the
// end of the row (VSeq::half returns n_halves for those) lies outside the buffer resource: the loads return zeros and
// fetch nothing, no select per row is needed (the rows of a sequence are whole 64-token blocks, so a half tile is
// inside or outside as a whole).
template <int D>
__device__ __forceinline__ void v_stream_issue_high(VHighPart<VStream<D>::HV> &t, const __amdgpu_buffer_rsrc_t rH, int half) {
    using S = VStream<D>;
    const int lane = threadIdx.x & 63;
    const int vo = (half * S::HT + lane / S::LPR) * D + (lane % S::LPR) * 16;
#pragma unroll
    for (int u = 0; u < S::HV; ++u) t.h[u] = __builtin_amdgcn_raw_buffer_load_b128(rH, vo + u * (S::TPL * D), 0, kStream);
}

template <int D>
__device__ __forceinline__ void v_stream_issue_probs(u32 *sb, const __amdgpu_buffer_rsrc_t rS, int half) {
    using S = VStream<D>;
    const int lane = threadIdx.x & 63;
    const int vo = (half * S::HT + lane / S::LPR) * 2;
#pragma unroll
    for (int u = 0; u < S::HV; ++u)
        sb[u] = (u32)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(rS, vo + u * (S::TPL * 2), 0, 0);
}

// requests half tile `half` (tokens half * HT ...) into ring slot k
template <int D, int NRING>
__device__ __forceinline__ void v_stream_issue(VRing<D, NRING> &ring, int k, const __amdgpu_buffer_rsrc_t rH,
                                               const __amdgpu_buffer_rsrc_t rS, int half) {
    // the probabilities first: loads return in order, and the fetch levels of a half tile are looked at one half
    // tile before its high bytes are needed
    v_stream_issue_probs<D>(ring.sb[k], rS, half);
    v_stream_issue_high<D>(ring.hi[k], rH, half);
}

// the first PF half tiles of the wave: before anything the caller has to do first (they depend on nothing but
// the probabilities, which the caller may still be writing: those are requested by v_stream_run, together with
// the high bytes of the half tiles PF .. NR - 2)
template <int D, int NR, int PF>
__device__ __forceinline__ void v_stream_prefetch(VRing<D, NR> &ring, const uint8_t *f8, int n_tokens, const VSeq &seq) {
    static_assert(PF <= NR - 1, "the ring keeps one slot for the half tile being multiplied");
    const __amdgpu_buffer_rsrc_t rH = make_rsrc(f8, (u32)n_tokens * D);
#pragma unroll
    for (int k = 0; k < PF; ++k) v_stream_issue_high<D>(ring.hi[k], rH, seq.half(k));
    __builtin_amdgcn_sched_barrier(0);
}

template <int D, bool REF, int NR, int PF>
__device__ __forceinline__ void v_stream_run(VRing<D, NR> &ring, const uint8_t *f8, const uint8_t *m4, const uint8_t *l4,
                                             int n_tokens, const unsigned short *s_row, unsigned char amin, const VSeq &seq,
                                             float *acc) {
    using S = VStream<D>;
    static_assert(NR % 2 == 0, "the two nibble buffers alternate with the ring slots");
    static_assert(NR >= 4, "the levels of half tile k + 1 are looked at before half tile k + NR - 1 is requested");
    constexpr int HV = S::HV;
    const __amdgpu_buffer_rsrc_t rH = make_rsrc(f8, (u32)n_tokens * D);
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(m4, (u32)n_tokens * (D / 2));
    const __amdgpu_buffer_rsrc_t rL = make_rsrc(l4, (u32)n_tokens * (D / 2));
    const __amdgpu_buffer_rsrc_t rS = make_rsrc(s_row, (u32)n_tokens * 2);
#pragma unroll
    for (int k = PF; k < NR - 1; ++k) v_stream_issue_high<D>(ring.hi[k], rH, seq.half(k));
    // probabilities of the half tiles requested so far
#pragma unroll
    for (int k = 0; k < NR - 1; ++k) v_stream_issue_probs<D>(ring.sb[k], rS, seq.half(k));
    VLowPart<HV> nib[2];
    bool fine_now = v_half_is_fine<REF, HV>(ring.sb[0], amin);
    if (fine_now) v_issue_half_ml<D, REF, HV>(nib[0], rM, rL, seq.half(0) * S::HT, n_tokens, ring.sb[0], amin);
    __builtin_amdgcn_sched_barrier(0);
    auto round = [&](int i0) {
#pragma unroll
        for (int k = 0; k < NR; ++k) {
            // nibble rows of the next half tile first, then the newest probabilities and high bytes
            const int kn = (k + 1) % NR;
            const bool fine_next = v_half_is_fine<REF, HV>(ring.sb[kn], amin);
            if (fine_next)
                v_issue_half_ml<D, REF, HV>(nib[(k + 1) & 1], rM, rL, seq.half(i0 + k + 1) * S::HT, n_tokens, ring.sb[kn], amin);
            v_stream_issue<D, NR>(ring, (k + NR - 1) % NR, rH, rS, seq.half(i0 + k + NR - 1));
            __builtin_amdgcn_sched_barrier(0);
            if (fine_now) v_compute_half<HV>(acc, ring.hi[k], nib[k & 1], ring.sb[k]);
            else v_compute_half_coarse<HV>(acc, ring.hi[k], ring.sb[k]);
            pin_accumulators(acc);
            __builtin_amdgcn_sched_barrier(0);
            fine_now = fine_next;
        }
    };
    // The first round stands outside the loop: the compiler derives the number of loads that may stay in flight at
    // a wait from every path that reaches it, and the path from the set-up above (fewer requests behind the one
    // waited for) would otherwise hold every round of the loop to the depth of the first.
    if (seq.left() > 0) {
        round(0);
        for (int i0 = NR; i0 < seq.left(); i0 += NR) round(i0);
    }
}

// Number of the wave's tokens below level 2: the probabilities of the wave's half tiles, 16 bytes per lane and load;
// for rows of at most 64 * 16 * 8 / 2 tokens per wave.
// LDSP: s_row is a copy of the row's probabilities in LDS (a caller that produced them in the same workgroup).
template <int D, bool LDSP = false>
__device__ __forceinline__ int v_stream_count_fine(const unsigned short *s_row, int n_tokens, unsigned char amin, const VSeq &seq) {
    using S = VStream<D>;
    constexpr int UPH = S::HT * 2 / 16;    // 16-byte units of probabilities per half tile
    const int lane = threadIdx.x & 63;
    const __amdgpu_buffer_rsrc_t rS = make_rsrc(s_row, (u32)n_tokens * 2);
    typedef short i16x2_t __attribute__((ext_vector_type(2)));
    typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
    const unsigned short a16 = (unsigned short)((unsigned)amin << 10);
    const u16x2_t a2 = {a16, a16};
    const i16x2_t c8 = {0x0800, 0x0800};
    int n = 0;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int f = lane + 64 * j, i = f / UPH, part = f % UPH;
        const bool on = seq.half(i) < seq.n_halves;
        u32x4 w;
        if constexpr (LDSP) w = on ? *reinterpret_cast<const u32x4 *>(s_row + seq.half(i) * S::HT + part * 8) : (u32x4){0u, 0u, 0u, 0u};
        else w = __builtin_amdgcn_raw_buffer_load_b128(rS, (seq.half(i) * S::HT + part * 8) * 2, 0, 0);
        const u32 ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            union { u32 u; u16x2_t v; } x;
            x.u = ww[k];
            union { u16x2_t u; i16x2_t s; } d;
            d.u = a2 - x.v;                                    // wraps like the reference's `short` arithmetic
            union { i16x2_t v; u32 u; } t;
            t.v = __builtin_elementwise_sub_sat(d.s, c8);      // negative <=> diff < 0x0800 <=> level < 2
            n += on ? __builtin_popcount((t.u >> 15) & 0x00010001u) : 0;
        }
    }
    return wave_sum_i32(n);
}

// The stream with every token multiplied at level 2 (high bytes only) and no look at the fetch levels: for a caller that
// does not know the row's threshold yet, or lists the tokens below level 2 some other way (VFineScan).
// One half tile in flight while one is multiplied; the probabilities come from LDS (probs_lds: the row's, token-indexed;
// probs_lds[zero_at ...] holds a half tile's worth of zeros, read for a half tile past the wave's share: a wave-uniform
// choice of the address instead of a branch around every read).
// prefetched: the share's first half tile has been requested into ring.hi[0] already (by the caller with
// v_stream_issue_high, or by the call for the share before this one through next_half).
// next_half: requested into ring.hi[0] when the share's last half tile is being multiplied (the first half tile of the
// share the wave takes next, so that the pipeline does not drain between the two calls), or n_halves for none.
// extra(i): called once per half tile, when the request of the next one is on its way (work that is to hide behind the
// stream's memory time).
struct NoExtra {
    __device__ __forceinline__ void operator()(int) const {}
};
template <int D, int RN, typename Extra = NoExtra>
__device__ __forceinline__ void v_stream_run_coarse(VRing<D, RN> &ring, const uint8_t *f8, int n_tokens,
                                                   const unsigned short *probs_lds, int zero_at, const VSeq &seq, bool prefetched,
                                                   int next_half, float *acc, Extra extra = Extra()) {
    using S = VStream<D>;
    constexpr int HV = S::HV;
    const int lane = threadIdx.x & 63, tl = lane / S::LPR;
    const __amdgpu_buffer_rsrc_t rH = make_rsrc(f8, (u32)n_tokens * D);
    if (seq.count <= 0) return;
    if (!prefetched) v_stream_issue_high<D>(ring.hi[0], rH, seq.half(0));
    __builtin_amdgcn_sched_barrier(0);
    auto round = [&](int i0) {
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            // (slot 0 after the share's last round: the next share's first half tile)
            const int ahead = (k == 1 && i0 + 2 >= seq.count) ? next_half : seq.half(i0 + k + 1);
            v_stream_issue_high<D>(ring.hi[k ^ 1], rH, ahead);
            __builtin_amdgcn_sched_barrier(0);
            extra(i0 + k);
            __builtin_amdgcn_sched_barrier(0);
            const int half = seq.half(i0 + k);
            // (a half tile past the wave's share: its high bytes came back as zeros, its probabilities count as zeros)
            const bool on = half < seq.n_halves;
            u32 sb[HV];
#pragma unroll
            for (int u = 0; u < HV; ++u) sb[u] = (u32)probs_lds[(on ? half * S::HT : zero_at) + tl + u * S::TPL];
            v_compute_half_coarse<HV>(acc, ring.hi[k], sb);
            pin_accumulators(acc);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // (the first round stands outside the loop: see v_stream_run)
    round(0);
    for (int i0 = 2; i0 < seq.count; i0 += 2) round(i0);
}

// The stream with every token read at its own fetch level, for rows where tokens below level 2 are frequent (flat
// attention).  The levels come from the row's probabilities in LDS (probs_lds, token-indexed) and the threshold, so a half
// tile's nibble rows are requested together with its high bytes, NR - 1 half tiles before it is multiplied; a row that is
// not needed is an out-of-range offset and fetches nothing.  extra(i): called once per half tile, between the request
// of the newest half tile and the multiplication of the oldest.
template <int D, int NR, typename Extra = NoExtra>
__device__ __forceinline__ void v_stream_run_levels(const uint8_t *f8, const uint8_t *m4, const uint8_t *l4, int n_tokens,
                                                   const unsigned short *probs_lds, int zero_at, unsigned char amin,
                                                   const VSeq &seq, float *acc, Extra extra = Extra()) {
    using S = VStream<D>;
    constexpr int HV = S::HV;
    static_assert(NR >= 2, "one half tile is multiplied while the others travel");
    if (seq.count <= 0) return;
    const int lane = threadIdx.x & 63, tl = lane / S::LPR;
    const __amdgpu_buffer_rsrc_t rH = make_rsrc(f8, (u32)n_tokens * D);
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(m4, (u32)n_tokens * (D / 2));
    const __amdgpu_buffer_rsrc_t rL = make_rsrc(l4, (u32)n_tokens * (D / 2));
    VHalfTile<HV> t[NR];
    u32 sb[NR][HV];
    auto issue = [&](VHalfTile<HV> &x, u32 *p, int half) {
        // (a half tile past the wave's share: probabilities of zero, level 2, nothing fetched)
        const bool on = half < seq.n_halves;
#pragma unroll
        for (int u = 0; u < HV; ++u) p[u] = (u32)probs_lds[(on ? half * S::HT : zero_at) + tl + u * S::TPL];
        v_stream_issue_high<D>(x, rH, half);
        v_issue_half_ml<D, false, HV>(x, rM, rL, half * S::HT, n_tokens, p, amin);
    };
#pragma unroll
    for (int k = 0; k < NR - 1; ++k) issue(t[k], sb[k], seq.half(k));
    __builtin_amdgcn_sched_barrier(0);
    auto round = [&](int i0) {
#pragma unroll
        for (int k = 0; k < NR; ++k) {
            issue(t[(k + NR - 1) % NR], sb[(k + NR - 1) % NR], seq.half(i0 + k + NR - 1));
            __builtin_amdgcn_sched_barrier(0);
            extra(i0 + k);
            __builtin_amdgcn_sched_barrier(0);
            v_compute_half<HV>(acc, t[k], sb[k]);
            pin_accumulators(acc);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // (the first round stands outside the loop: see v_stream_run)
    round(0);
    for (int i0 = NR; i0 < seq.count; i0 += NR) round(i0);
}

// Lists the tokens below level 2 of a wave's shares a and b (in that order) from the row's probabilities in LDS, 64 tokens
// per step: list[count ...] gets (token | probability bits << 16).  A token with probability zero never counts.
template <int D>
struct VFineScan {
    using S = VStream<D>;
    static constexpr int TPI = 64 / S::HT;       // half tiles per step
    const unsigned short *probs_lds;
    unsigned char amin;
    VSeq a, b;
    int pos = 0;
    __device__ __forceinline__ bool done() const { return pos >= a.count + b.count; }
    __device__ __forceinline__ int steps_left() const { return (a.count + b.count - pos + TPI - 1) / TPI; }
    __device__ __forceinline__ void step(u32 *list, int &count) {
        const int lane = threadIdx.x & 63;
        const int i = pos + lane / S::HT;
        const int half = i < a.count ? a.start + i * a.stride : b.half(i - a.count);
        const bool on = half < a.n_halves;
        const int tok = half * S::HT + lane % S::HT;
        const u32 pb = on ? (u32)probs_lds[tok] : 0u;
        VListed<D>::append(list, count, pb != 0u && v_level(amin, (unsigned short)pb) < 2, tok, pb);
        pos += TPI;
    }
};

// Folds the token lanes of a wave together and adds the 4 waves of the workgroup:
// out[d] (d < D) = sum over all 256 lanes of their acc for channel d.  wave_part: LDS [4][D].
template <int D, int NW = 4>
__device__ __forceinline__ void v_fold_lanes(float *acc, float (*wave_part)[D]) {
    // leaves wave_part[wave][d] = this wave's sum for channel d (caller synchronises)
    constexpr int LPR = D / 16;
    constexpr int NV = LPR == 16 ? 4 : (LPR == 8 ? 2 : 1);
    const int lane = threadIdx.x & 63, wave = wave_index();
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
}

template <int D>
__device__ __forceinline__ void v_fold_workgroup(float *acc, float (*wave_part)[D], float *out) {
    constexpr int LPR = D / 16;
    constexpr int NV = LPR == 16 ? 4 : (LPR == 8 ? 2 : 1);   // sums left per lane
    const int lane = threadIdx.x & 63, wave = wave_index();
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
    const __amdgpu_buffer_rsrc_t rO = make_rsrc(out, (u32)D * 4);
    for (int d = threadIdx.x; d < D; d += 256)
        store_f32_device(rO, d * 4, (wave_part[0][d] + wave_part[1][d]) + (wave_part[2][d] + wave_part[3][d]));
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
    return bpw;
}


inline int k256_blocks_per_wave(int B, int H, int n_blocks) {
    // a wave streams 64 KiB per 256-token block: one block per wave unless that makes more than ~16 k waves
    int bpw = 1;
    while (bpw < 4 && (int64_t)B * H * ((n_blocks + bpw * 2 - 1) / (bpw * 2)) >= 8192) bpw *= 2;
    return bpw;
}

}  // namespace akv
