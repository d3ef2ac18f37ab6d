// Grouped-query K and V passes on the matrix cores.
//
// With G query heads per KV head the passes are skinny matrix products (tokens x channels times channels x G):
// on the vector ALUs every query head repeats the unpack-and-multiply of the shared tile (2.5 vector operations
// per query-head element), which makes the pass ALU-bound from G = 4 on.  Here the shared tile is unpacked ONCE
// into fp16 MFMA operands and v_mfma_f32_16x16x16_f16 does the multiply for up to 16 query heads (columns) with
// fp32 accumulation: fp16 x fp16 products are exact in fp32, so results differ from the vector kernels only in
// summation order.
//
// Per-head fetch levels (K: extension/csrc/K_cache.cu:211,249-252; V: extension/csrc/V_cache.cu:195-197,250-253)
// stay exact.  A plane row is fetched at the finest level any head of the group asks for ("union level"); the
// operand A holds the values at that level.  A head with a coarser level needs the value with its low bits
// replaced (0x8 / 0x80): sub1(A) or sub2(A), one and-or per register.  Three MFMAs -- A, sub1(A), sub2(A) against x where
// the head's level is 0, 1, 2 and zero elsewhere -- give every head exactly its own levels (mfma_levels).  Where a
// tile has already been multiplied at level 2 throughout, what is missing is A - sub2(A) (level 0) or
// sub1(A) - sub2(A) (level 1): differences that are exact in fp16 (same sign, exponent and upper mantissa), two MFMAs
// (kt_correct).
#include "akv_step.h"

namespace akv {

typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f16x4 as_f16x4(u32 lo, u32 hi) {
    union { u32 u[2]; f16x4 v; } x;
    x.u[0] = lo;
    x.u[1] = hi;
    return x.v;
}
__device__ __forceinline__ f16x2 as_f16x2(u32 w) {
    union { u32 u; f16x2 v; } x;
    x.u = w;
    return x.v;
}
__device__ __forceinline__ u32 as_u32(f16x2 v) {
    union { u32 u; f16x2 v; } x;
    x.v = v;
    return x.u;
}
// packed pair of fp16 values minus the same pair with the low bits replaced: exact
__device__ __forceinline__ u32 low_bits_excess(u32 w, u32 keep, u32 put) {
    return as_u32(as_f16x2(w) - as_f16x2((w & keep) | put));
}

// the substitution bits of levels 1 and 2 for a pair of fp16 values, kept in vector registers
struct LevelPuts {
    u32 put1 = 0x00080008u, put2 = 0x00800080u;
    __device__ __forceinline__ void pin() { asm volatile("" : "+v"(put1), "+v"(put2)); }
};

// acc += A x B0 + sub1(A) x B1 + sub2(A) x B2: B0 / B1 / B2 hold x where the head reads the element at level 0 / 1 / 2
// and zero elsewhere (every plane read: only A x B0)
template <bool REF>
__device__ __forceinline__ void mfma_levels(f32x4 &acc, u32 a_lo, u32 a_hi, f16x4 b0, f16x4 b1, f16x4 b2, u32 put1,
                                            u32 put2) {
    // put1 = 0x00080008, put2 = 0x00800080 in vector registers (LevelPuts): (w & keep) | put is then one v_and_or_b32
    // (an instruction takes one literal constant)
    acc = __builtin_amdgcn_mfma_f32_16x16x16f16(as_f16x4(a_lo, a_hi), b0, acc, 0, 0, 0);
    if (!REF) {
        acc = __builtin_amdgcn_mfma_f32_16x16x16f16(as_f16x4((a_lo & 0xFFF0FFF0u) | put1, (a_hi & 0xFFF0FFF0u) | put1), b1, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x16f16(as_f16x4((a_lo & 0xFF00FF00u) | put2, (a_hi & 0xFF00FF00u) | put2), b2, acc, 0, 0, 0);
    }
}

// ------------------------------------------------------------------------------------------------
// K pass.  A wave takes tasks of SL/4 blocks (SL = slots per lane: 16, 8 or 4).  Lane l: token set ts = l % 16 =
// (block of the task, piece of SL slots of its 64), channel residue cs = l / 16; per channel group kg (16
// channels) it loads the SL slots of the channels 16 kg + 4 r + cs (r < 4).  In the MFMA the token sets are the
// rows, (cs, r) the contraction index, the query heads the columns: the partial sums over channels that the
// vector kernel folds with 15 shuffles per head are summed inside the instruction.  Lane (j, ig) ends up with
// the scores of token sets 4 ig .. 4 ig + 3 for query head j.
// Smaller SL: fewer accumulators (4 SL registers) and smaller tiles, hence more waves per SIMD and more tiles in
// flight per wave at the same register budget -- what hides the several-microsecond loaded HBM latency -- at the
// price of narrower loads.
// grid (ceil(tasks / (4 * tasks_per_wave)), Hkv, B), 256 threads.
// ------------------------------------------------------------------------------------------------
template <int SL>
struct KTaskTile {   // one channel group: 4 channels x SL slots per lane
    u32 h[4][SL / 4];
    u32 m[4][(SL + 7) / 8], l[4][(SL + 7) / 8];
};

template <int NB>
__device__ __forceinline__ void load_bytes(u32 *dst, const __amdgpu_buffer_rsrc_t r, int off) {
    if constexpr (NB == 16) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, off, 00, kStream);
        dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w;
    } else if constexpr (NB == 8) {
        const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(r, off, 00, kStream);
        dst[0] = v.x; dst[1] = v.y;
    } else if constexpr (NB == 4) {
        dst[0] = __builtin_amdgcn_raw_buffer_load_b32(r, off, 00, kStream);
    } else {
        dst[0] = (u32)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(r, off, 00, kStream);
    }
}

// KSH: log2 of 64-token blocks per K plane block (0: plane blocks of 64 tokens, 2: of 256).  blk counts 64-token
// blocks either way; in a 256-token plane block a channel's row holds the slots of four of them side by side.
template <int D, int SL, int KSH>
__device__ __forceinline__ void kt_issue(KTaskTile<SL> &t, const __amdgpu_buffer_rsrc_t rH, const __amdgpu_buffer_rsrc_t rM,
                                         const __amdgpu_buffer_rsrc_t rL, int blk, int kg, u32 need_mid, u32 need_last) {
    constexpr int PB = 64 / SL;   // pieces per block
    constexpr int KB = 64 << KSH;
    const int lane = threadIdx.x & 63;
    const int piece = (lane & 15) % PB, cs = lane >> 4;
    const int kblk = blk >> KSH, sub = blk & ((1 << KSH) - 1);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int c = 16 * kg + 4 * r + cs;
        load_bytes<SL>(t.h[r], rH, kblk * (D * KB) + c * KB + sub * 64 + piece * SL);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int c = 16 * kg + 4 * r + cs;
        const int off = kblk * (D * KB / 2) + c * (KB / 2) + sub * 32 + piece * (SL / 2);
        load_bytes<SL / 2>(t.m[r], rM, ((need_mid >> (4 * kg + r)) & 1u) ? off : kSkip);
        load_bytes<SL / 2>(t.l[r], rL, ((need_last >> (4 * kg + r)) & 1u) ? off : kSkip);
    }
}

template <bool REF, int SL>
__device__ __forceinline__ void kt_compute(f32x4 *acc, const KTaskTile<SL> &t, int kg, u32 need_mid, u32 need_last, f16x4 b0,
                                           f16x4 b1, f16x4 b2, const LevelPuts &lp) {
    constexpr int NX = (SL + 7) / 8;       // units of 8 slots (one unit of 4 for SL == 4)
    constexpr int NP = SL == 4 ? 2 : 4;    // slot pairs per unit
#pragma unroll
    for (int x = 0; x < NX; ++x) {
        u32 w[4][4];                 // [r][pair]: slots 8x + (0,2), (1,3), (4,6), (5,7) of channel r
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const bool mid = (need_mid >> (4 * kg + r)) & 1u, last = (need_last >> (4 * kg + r)) & 1u;
            const u32 cm = mid ? 0u : 0x88888888u;               // union level 2: low byte 0x80
            const u32 cl = (mid && !last) ? 0x88888888u : 0u;    // union level 1: last nibble 0x8
            u32 E, O;
            split_even_odd(t.m[r][x] | cm, t.l[r][x] | cl, E, O);
            const u32 Ha = t.h[r][SL == 4 ? 0 : 2 * x];
            w[r][0] = __builtin_amdgcn_perm(Ha, E, 0x06010400u);
            w[r][1] = __builtin_amdgcn_perm(Ha, O, 0x07010500u);
            if constexpr (SL != 4) {
                const u32 Hb = t.h[r][2 * x + 1];
                w[r][2] = __builtin_amdgcn_perm(Hb, E, 0x06030402u);
                w[r][3] = __builtin_amdgcn_perm(Hb, O, 0x07030502u);
            }
        }
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int s0 = 8 * x + (p & 1) + 4 * (p >> 1);        // the pair holds slots s0 and s0 + 2
            // 2x2 transposes: (channel r, slot pair) -> (slot, channel pair)
            const u32 a01_s0 = __builtin_amdgcn_perm(w[1][p], w[0][p], 0x05040100u);
            const u32 a23_s0 = __builtin_amdgcn_perm(w[3][p], w[2][p], 0x05040100u);
            const u32 a01_s2 = __builtin_amdgcn_perm(w[1][p], w[0][p], 0x07060302u);
            const u32 a23_s2 = __builtin_amdgcn_perm(w[3][p], w[2][p], 0x07060302u);
            mfma_levels<REF>(acc[s0], a01_s0, a23_s0, b0, b1, b2, lp.put1, lp.put2);
            mfma_levels<REF>(acc[s0 + 2], a01_s2, a23_s2, b0, b1, b2, lp.put1, lp.put2);
        }
    }
}

// Set-up of the K pass, once per (batch, KV head) instead of once per wave: lane (j, kq) = (l % 16, l / 16) takes
// query head j of the group at the channels 16 kg + 4 r + kq and leaves, for the K-pass lane of the same index,
// 2 KG words of q (packed fp16 pairs r = 0,1 / 2,3 per channel group) and 4 words of level bits (bit 4 kg + r):
// this head's level is 1 / is 2, and -- OR-ed over the heads of the group -- the mid / last plane row of the
// channel is fetched.  One wave per (batch, KV head): mfma_k_prepare (akv_step.h), run by this
// kernel (grid (B * Hkv), 64 threads) or, with per-sequence lengths, by extra workgroups of the step's first kernel.
template <int D, bool REF>
__global__ __launch_bounds__(64) void mfma_k_prepare_kernel(const uint8_t *__restrict__ kcm, const unsigned short *__restrict__ q,
                                                           const unsigned short *__restrict__ k_new, u32 *__restrict__ prep,
                                                           uint8_t *__restrict__ levels_out, StepGeom geo) {
    mfma_k_prepare<D, REF>(kcm, q, k_new, prep, levels_out, geo, (int)blockIdx.x);
}

// The same for a tile whose rows are all used at level 2 by every head (only the high bytes were fetched): the low
// byte is the constant 0x80 and there is nothing to correct.
template <int SL>
__device__ __forceinline__ void kt_compute_coarse(f32x4 *acc, const KTaskTile<SL> &t, f16x4 b0) {
    constexpr int NX = (SL + 7) / 8;
    constexpr int NP = SL == 4 ? 2 : 4;
    const u32 c80 = 0x80808080u;
#pragma unroll
    for (int x = 0; x < NX; ++x) {
        u32 w[4][4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const u32 Ha = t.h[r][SL == 4 ? 0 : 2 * x];
            w[r][0] = __builtin_amdgcn_perm(Ha, c80, 0x06010400u);
            w[r][1] = __builtin_amdgcn_perm(Ha, c80, 0x07010500u);
            if constexpr (SL != 4) {
                const u32 Hb = t.h[r][2 * x + 1];
                w[r][2] = __builtin_amdgcn_perm(Hb, c80, 0x06030402u);
                w[r][3] = __builtin_amdgcn_perm(Hb, c80, 0x07030502u);
            }
        }
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int s0 = 8 * x + (p & 1) + 4 * (p >> 1);
            const u32 a01_s0 = __builtin_amdgcn_perm(w[1][p], w[0][p], 0x05040100u);
            const u32 a23_s0 = __builtin_amdgcn_perm(w[3][p], w[2][p], 0x05040100u);
            const u32 a01_s2 = __builtin_amdgcn_perm(w[1][p], w[0][p], 0x07060302u);
            const u32 a23_s2 = __builtin_amdgcn_perm(w[3][p], w[2][p], 0x07060302u);
            acc[s0] = __builtin_amdgcn_mfma_f32_16x16x16f16(as_f16x4(a01_s0, a23_s0), b0, acc[s0], 0, 0, 0);
            acc[s0 + 2] = __builtin_amdgcn_mfma_f32_16x16x16f16(as_f16x4(a01_s2, a23_s2), b0, acc[s0 + 2], 0, 0, 0);
        }
    }
}

// The two correction products alone: acc += C2 x B2 + C1 x B1 (operands as in mfma_levels)
__device__ __forceinline__ void mfma_corrections(f32x4 &acc, u32 a_lo, u32 a_hi, f16x4 b1, f16x4 b2, u32 put1, u32 put2) {
    acc = __builtin_amdgcn_mfma_f32_16x16x16f16(
        as_f16x4(low_bits_excess(a_lo, 0xFF00FF00u, put2), low_bits_excess(a_hi, 0xFF00FF00u, put2)), b2, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x16f16(
        as_f16x4(low_bits_excess(a_lo, 0xFFF0FFF0u, put1), low_bits_excess(a_hi, 0xFFF0FFF0u, put1)), b1, acc, 0, 0, 0);
}

// What a tile that was multiplied at level 2 throughout still lacks: with A the values at the union level,
// value_at_level - value_at_level_2 = C2 (level 0) or C2 - C1 (level 1), hence acc += C2 x (x [level < 2]) +
// C1 x (-x [level == 1]).  need_mid / need_last: bit r of the lane's row r (as in kt_compute with kg = 0).
template <int SL>
__device__ __forceinline__ void kt_correct(f32x4 *acc, const KTaskTile<SL> &t, u32 need_mid, u32 need_last, f16x4 b1, f16x4 b2,
                                           const LevelPuts &lp) {
    constexpr int NX = (SL + 7) / 8;
    constexpr int NP = SL == 4 ? 2 : 4;
#pragma unroll
    for (int x = 0; x < NX; ++x) {
        u32 w[4][4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const bool mid = (need_mid >> r) & 1u, last = (need_last >> r) & 1u;
            const u32 cm = mid ? 0u : 0x88888888u;
            const u32 cl = (mid && !last) ? 0x88888888u : 0u;
            u32 E, O;
            split_even_odd(t.m[r][x] | cm, t.l[r][x] | cl, E, O);
            const u32 Ha = t.h[r][SL == 4 ? 0 : 2 * x];
            w[r][0] = __builtin_amdgcn_perm(Ha, E, 0x06010400u);
            w[r][1] = __builtin_amdgcn_perm(Ha, O, 0x07010500u);
            if constexpr (SL != 4) {
                const u32 Hb = t.h[r][2 * x + 1];
                w[r][2] = __builtin_amdgcn_perm(Hb, E, 0x06030402u);
                w[r][3] = __builtin_amdgcn_perm(Hb, O, 0x07030502u);
            }
        }
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int s0 = 8 * x + (p & 1) + 4 * (p >> 1);
            const u32 a01_s0 = __builtin_amdgcn_perm(w[1][p], w[0][p], 0x05040100u);
            const u32 a23_s0 = __builtin_amdgcn_perm(w[3][p], w[2][p], 0x05040100u);
            const u32 a01_s2 = __builtin_amdgcn_perm(w[1][p], w[0][p], 0x07060302u);
            const u32 a23_s2 = __builtin_amdgcn_perm(w[3][p], w[2][p], 0x07060302u);
            mfma_corrections(acc[s0], a01_s0, a23_s0, b1, b2, lp.put1, lp.put2);
            mfma_corrections(acc[s0 + 2], a01_s2, a23_s2, b1, b2, lp.put1, lp.put2);
        }
    }
}

template <int D, bool REF, int SL, int AHEAD, int KSH>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(SL == 8 && AHEAD == 3 ? 3 : 1))) void mfma_k_pass_kernel(
    const uint8_t *__restrict__ first_8, const uint8_t *__restrict__ mid_4, const uint8_t *__restrict__ last_4,
    const u32 *__restrict__ prep, unsigned short *__restrict__ scores, StepGeom geo, int tasks_per_wave, float scale,
    u32 scores_bytes) {
    constexpr int CB = 64;
    constexpr int KG = D / 16;     // channel groups
    constexpr int PB = 64 / SL;    // pieces (token sets) per block
    constexpr int NBT = 16 / PB;   // blocks per task
    static_assert(KG % (AHEAD + 1) == 0, "the tile ring is rotated by unrolling");
    const int lane = threadIdx.x & 63, wave = wave_index();
    int chunk, hkv, b;
    if (!step_block(geo, chunk, hkv, b)) return;
    const int G = geo.G;
    const int bh_kv = b * geo.Hkv + hkv;
    const int64_t bh0 = (int64_t)b * geo.Hq + hkv * G;
    int R, nrest;
    seq_state(geo, b, R, nrest);
    const int n_blocks = R / CB;
    const int n_tasks = (n_blocks + NBT - 1) / NBT;
    const int first_task = (chunk * 4 + wave) * tasks_per_wave;
    const int end_task = min(first_task + tasks_per_wave, n_tasks);
    if (first_task >= n_tasks) return;     // past the end of this sequence (no barrier in this kernel)

    // geo.n_max_blocks counts K plane blocks (of 64 << KSH tokens); the resources end with the last one that holds tokens
    constexpr int KB = CB << KSH;
    const int n_kblocks = (n_blocks + (1 << KSH) - 1) >> KSH;
    const int64_t plane_off = (int64_t)bh_kv * geo.n_max_blocks * (D * (KB / 2));
    const __amdgpu_buffer_rsrc_t rH = make_rsrc(first_8 + plane_off * 2, (u32)n_kblocks * (D * KB));
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(mid_4 + plane_off, (u32)n_kblocks * (D * KB / 2));
    const __amdgpu_buffer_rsrc_t rL = make_rsrc(last_4 + plane_off, (u32)n_kblocks * (D * KB / 2));
    const __amdgpu_buffer_rsrc_t rS = make_rsrc(scores, scores_bytes);
    const int blk_sel = (lane & 15) / PB;

    // what mfma_k_prepare_kernel left for this lane
    const int j = lane & 15;
    const bool head = j < G;
    u32 qp[KG][2];
    u32 lv1, lv2, need_mid, need_last;
    {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(prep + ((int64_t)bh_kv * 64 + lane) * (2 * KG + 4));
#pragma unroll
        for (int i = 0; i < KG / 2; ++i) {
            const u32x4 v = src[i];
            qp[2 * i][0] = v.x; qp[2 * i][1] = v.y; qp[2 * i + 1][0] = v.z; qp[2 * i + 1][1] = v.w;
        }
        const u32x4 v = src[KG / 2];
        lv1 = v.x; lv2 = v.y; need_mid = v.z; need_last = v.w;
    }

    LevelPuts puts;
    puts.pin();
    // Software pipeline: AHEAD channel-group tiles in flight while one is multiplied.
    KTaskTile<SL> t[AHEAD + 1];
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) kt_issue<D, SL, KSH>(t[i], rH, rM, rL, first_task * NBT + blk_sel, i, need_mid, need_last);
    __builtin_amdgcn_sched_barrier(0);
    for (int task = first_task; task < end_task; ++task) {
        f32x4 acc[SL];
#pragma unroll
        for (int i = 0; i < SL; ++i) acc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
        // the masks derived from these words are cheap to rebuild and would otherwise be kept in ~100 registers
        // across the loop: hide their loop invariance from the compiler
        asm volatile("" : "+v"(need_mid), "+v"(need_last), "+v"(lv1), "+v"(lv2));
        const int blk = task * NBT + blk_sel;
        const int next_blk = (task + 1 < end_task ? task + 1 : n_tasks) * NBT + blk_sel;   // past the end: nothing is fetched
#pragma unroll
        for (int kg = 0; kg < KG; ++kg) {
            const int kn = kg + AHEAD;
            kt_issue<D, SL, KSH>(t[kn % (AHEAD + 1)], rH, rM, rL, kn < KG ? blk : next_blk, kn % KG, need_mid, need_last);
            __builtin_amdgcn_sched_barrier(0);
            const u32 m1a = ((lv1 >> (4 * kg)) & 1u ? 0xFFFFu : 0u) | ((lv1 >> (4 * kg + 1)) & 1u ? 0xFFFF0000u : 0u);
            const u32 m1b = ((lv1 >> (4 * kg + 2)) & 1u ? 0xFFFFu : 0u) | ((lv1 >> (4 * kg + 3)) & 1u ? 0xFFFF0000u : 0u);
            const u32 m2a = ((lv2 >> (4 * kg)) & 1u ? 0xFFFFu : 0u) | ((lv2 >> (4 * kg + 1)) & 1u ? 0xFFFF0000u : 0u);
            const u32 m2b = ((lv2 >> (4 * kg + 2)) & 1u ? 0xFFFFu : 0u) | ((lv2 >> (4 * kg + 3)) & 1u ? 0xFFFF0000u : 0u);
            const u32 qa = qp[kg][0], qb = qp[kg][1];
            kt_compute<REF, SL>(acc, t[kg % (AHEAD + 1)], kg, need_mid, need_last, as_f16x4(qa & ~(m1a | m2a), qb & ~(m1b | m2b)),
                                as_f16x4(qa & m1a, qb & m1b), as_f16x4(qa & m2a, qb & m2b), puts);
            __builtin_amdgcn_sched_barrier(0);
        }
        // lane (j, ig): acc[s][r] = score of slot s of token set 4 ig + r for query head j.  Plain stores throughout: the
        // scores are read by the step's next kernel.
        if constexpr (SL == 16) {
            // A head lane (j, ig) holds the 64 scores of block 4 task + ig for its head: one 128-byte line of the head's score
            // row.  Stored from there, an instruction scatters sixteen 16-byte pieces over sixteen lines, and the 19 MB of
            // scores cost the pass 7 us of 54 at batch 32, 32 over 8 heads, lengths 2048 to 8192 (47.1 us with the stores
            // dropped; written through at device scope, as they were first, 56.7).  The lines go through LDS instead
            // -- line (ig, head) at (ig * G + j) * 128 -- and eight consecutive lanes store a whole line, 16 bytes each:
            // 53.2 us and 9.5 MiB written, whatever the cache policy of the stores.  (The rest is what 10 MB of writes
            // cost next to the reads: 47.7 us with the same stores aimed at a region that stays in L2.)
            __shared__ __attribute__((aligned(16))) u32x4 lines[4][64 * 8];   // per wave: up to 4 x 16 lines of 8 pieces
            u32x4 *mine = lines[wave];
            if (head) {
                const int lam = (lane >> 4) * G + j;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    u32 pk[8];
#pragma unroll
                    for (int sl = 0; sl < 16; sl += 2)
                        pk[sl >> 1] = (u32)float_to_half_bits(acc[sl][r] * scale) | ((u32)float_to_half_bits(acc[sl + 1][r] * scale) << 16);
                    mine[lam * 8 + 2 * r] = (u32x4){pk[0], pk[1], pk[2], pk[3]};
                    mine[lam * 8 + 2 * r + 1] = (u32x4){pk[4], pk[5], pk[6], pk[7]};
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // the lines are read by other lanes of the wave
            const int n_lines = 4 * G;
            for (int s0 = 0; s0 * 8 < n_lines; ++s0) {
                const int lam = s0 * 8 + (lane >> 3);
                const int ig = lam / G, h = lam - ig * G;
                const int out_blk = task * NBT + ig;
                const bool store = lam < n_lines && out_blk < n_blocks;
                const u32x4 v = mine[lam * 8 + (lane & 7)];
                const int off = store ? (int)(((bh0 + h) * geo.row_stride + out_blk * CB) * 2) + (lane & 7) * 16 : kSkip;
                __builtin_amdgcn_raw_buffer_store_b128(v, rS, off, 0, 0);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // (read before the next task's lines are written)
        } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int ts = 4 * (lane >> 4) + r;
            const int out_blk = task * NBT + ts / PB;
            const bool store = head && out_blk < n_blocks;
            u32 pk[SL / 2];
#pragma unroll
            for (int sl = 0; sl < SL; sl += 2)
                pk[sl >> 1] = (u32)float_to_half_bits(acc[sl][r] * scale) | ((u32)float_to_half_bits(acc[sl + 1][r] * scale) << 16);
            const int off = store ? (int)(((bh0 + j) * geo.row_stride + out_blk * CB + (ts % PB) * SL) * 2) : kSkip;
            if constexpr (SL == 4) {
                __builtin_amdgcn_raw_buffer_store_b64((u32x2){pk[0], pk[1]}, rS, off, 0, 0);
            } else {
                __builtin_amdgcn_raw_buffer_store_b128((u32x4){pk[0], pk[1], pk[2], pk[3]}, rS, off, 0, 0);
            }
        }
        }
    }
}

// ---- host ------------------------------------------------------------------------------------------
template <int D>
int launch_mfma_k_pass(const uint8_t *f8, const uint8_t *m4, const uint8_t *l4, const uint8_t *kcm,
                       const unsigned short *q, const unsigned short *k_new, unsigned short *scores,
                       uint8_t *levels_out, u32 *prep, const StepGeom &geo, int B, int n_blocks, bool ref, float scale,
                       hipStream_t st, PassShape *shape_only, bool prepared) {
    // Slots per lane.  K blocks of 256 tokens: 16, so that the 16 lanes of a token-set group read a channel's whole row
    // of a block (256 B of first_8, 128 B of a nibble plane); measured at batch 32, 32 over 8 heads, lengths 2048..8192:
    // 62.5 us, against 78 with 8 slots per lane (half rows) and 68.8 with blocks of 64 tokens and 8 slots.  Three tiles
    // ahead instead of one (one wave per SIMD instead of two) measured 75.7 us, two tasks per wave 69.1.
    const int sl = geo.kb == 256 ? 16 : 8;
    const int nbt = sl / 4;
    const int n_tasks = (n_blocks + nbt - 1) / nbt;
    int tpw = 1;
    while (tpw < 8 && (int64_t)B * geo.Hkv * ((n_tasks + 8 * tpw - 1) / (8 * tpw)) * 4 >= 32768) tpw *= 2;
    if (shape_only != nullptr) {
        *shape_only = PassShape{(n_tasks + 4 * tpw - 1) / (4 * tpw), geo.Hkv, 4 * tpw * nbt * 64};
        return AKV_OK;
    }
    const int64_t scores_bytes = (int64_t)B * geo.Hq * geo.row_stride * 2;
    if (scores_bytes >= ((int64_t)1 << 31)) {
        set_error("decode_step: score rows of %lld bytes exceed the 2 GiB the grouped K pass addresses", (long long)scores_bytes);
        return AKV_ERR_INVALID;
    }
    if (!prepared) {
        if (ref)
            hipLaunchKernelGGL((mfma_k_prepare_kernel<D, true>), dim3(B * geo.Hkv), dim3(64), 0, st, kcm, q, k_new, prep, levels_out, geo);
        else
            hipLaunchKernelGGL((mfma_k_prepare_kernel<D, false>), dim3(B * geo.Hkv), dim3(64), 0, st, kcm, q, k_new, prep, levels_out, geo);
        int rc = check_launch("decode_step(mfma k_prepare)");
        if (rc != AKV_OK) return rc;
    }
    dim3 grid((n_tasks + 4 * tpw - 1) / (4 * tpw), geo.Hkv, B);
#define AKV_MK(RF, SLL, AH, KSH)                                                                                     \
    hipLaunchKernelGGL((mfma_k_pass_kernel<D, RF, SLL, AH, KSH>), grid, dim3(256), 0, st, f8, m4, l4, prep, scores, geo, \
                       tpw, scale, (u32)scores_bytes)
    // 256-token blocks: 16 slots per lane, one tile ahead; 64-token blocks: 8 slots per lane, three tiles ahead
    if (geo.kb == 256) { if (ref) AKV_MK(true, 16, 1, 2); else AKV_MK(false, 16, 1, 2); }
    else { if (ref) AKV_MK(true, 8, 3, 0); else AKV_MK(false, 8, 3, 0); }
#undef AKV_MK
    return check_launch("decode_step(mfma k_pass)");
}

// ------------------------------------------------------------------------------------------------
// V pass.  out[j][c] = sum over tokens of p_j[t] * v_level_j(t)[t][c]: rows = channels, contraction = tokens,
// columns = query heads.  Lane l: channel piece i = l % 16 (D/16 channels), token residue tg = l / 16; a step is
// 16 tokens (token = step base + 4 tg + u, u < 4 loads), a tile is the lane's D/16 channels of its 4 tokens -- the
// same register shape as a K tile with slots and channels exchanged, so the unpacking (kt_compute) is shared.
// The fetch level depends on the token: lane (j, tg) holds the probabilities of head j for the 4 tokens of its
// lane group and works out their levels; the OR over the 16 lanes of the group gives the planes to fetch for
// exactly the tokens the group's lanes load.  Lane (j, ig) ends up with 4 x D/16 output channels of head j.
// A wave walks tokens_per_wave tokens in macro steps of 64 (4 tiles, three in flight while one is multiplied);
// the probabilities are requested two macro steps ahead so that waiting for them never waits for a tile.
// grid (n_chunks, Hkv, B), 256 threads.
// ------------------------------------------------------------------------------------------------
template <int D>
__device__ __forceinline__ void vt_issue(KTaskTile<D / 16> &t, const __amdgpu_buffer_rsrc_t rH, const __amdgpu_buffer_rsrc_t rM,
                                         const __amdgpu_buffer_rsrc_t rL, int lane_h, int lane_m, int step_base, bool valid,
                                         bool fine, u32 need_mid, u32 need_last) {
    // lane_h / lane_m: byte offsets of the lane's piece in the row of token 4 tg; step_base and valid are wave-uniform
    constexpr int CPP = D / 16;
    const int oh = valid ? lane_h + step_base * D : kSkip, om = lane_m + step_base * (D / 2);
#pragma unroll
    for (int u = 0; u < 4; ++u) load_bytes<CPP>(t.h[u], rH, oh + u * D);
    if (!fine) return;   // wave-uniform: no lane of the wave fetches a nibble row of this step
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        load_bytes<CPP / 2>(t.m[u], rM, (valid && ((need_mid >> u) & 1u)) ? om + u * (D / 2) : kSkip);
        load_bytes<CPP / 2>(t.l[u], rL, (valid && ((need_last >> u) & 1u)) ? om + u * (D / 2) : kSkip);
    }
}

// What a lane needs for one macro step (64 tokens = 4 steps of 16): the probabilities of its head for its 16
// tokens (4 per step), their levels as bit sets (bit 4 s + u), and the planes its lane group fetches.
struct VMacroOps {
    u32x2 p[4];           // step s: tokens 4 kq + 0..3 of the step, packed fp16 pairs
    u32 lv1, lv2;         // this head's level of the token is 1 / 2
    u32 need;             // bits 0..15: mid row fetched, bits 16..31: last row fetched (union over the heads)
};

typedef short i16x2 __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
// packed 16-bit a - b with wrap-around, read as signed
__device__ __forceinline__ i16x2 wrap_diff16(u16x2 a, u32 b) {
    union { u32 u; u16x2 v; } x;
    x.u = b;
    union { u16x2 u; i16x2 s; } d;
    d.u = a - x.v;
    return d.s;
}

// a2: amin << 10 in both halves; lanes without a head pass 0x0800 and probabilities of zero (no token below level 2).
template <bool REF>
__device__ __forceinline__ void v_macro_ops(VMacroOps &o, const u32x2 *p, u16x2 a2, bool head) {
    u32 mid = 0, last = 0;
#pragma unroll
    for (int sidx = 0; sidx < 4; ++sidx) o.p[sidx] = p[sidx];
    if (REF) {
        mid = last = head ? 0xffffu : 0u;
    } else {
        // 16-bit differences of two tokens at a time (they wrap like the reference's `short` arithmetic,
        // extension/csrc/V_cache.cu:195-197,211); level < 2 <=> diff < 0x0800, level 0 <=> diff < 0x0400, read off the
        // sign of a saturating subtraction.  Word w = 2 s + (0: tokens 0,1 | 1: tokens 2,3 of step s) leaves the flag
        // of its first token in bit 2 w and of its second in bit 16 + 2 w.
        const i16x2 c8 = {0x0800, 0x0800}, c4 = {0x0400, 0x0400};
        i16x2 d[8];
        u32 t8[8], any8 = 0;
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            d[w] = wrap_diff16(a2, (w & 1) ? p[w >> 1].y : p[w >> 1].x);
            union { i16x2 v; u32 u; } t;
            t.v = __builtin_elementwise_sub_sat(d[w], c8);
            t8[w] = t.u;
            any8 |= t.u;
        }
        // nearly always no lane of the wave has a token below level 2 in these 64 tokens: nothing else to work out
        if (__builtin_amdgcn_ballot_w64((any8 & 0x80008000u) != 0u) == 0ull) {
            o.lv1 = 0;
            o.lv2 = 0xffffu;
            o.need = 0;
            return;
        }
        u32 acc8 = 0, acc4 = 0;
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            union { i16x2 v; u32 u; } t4;
            t4.v = __builtin_elementwise_sub_sat(d[w], c4);
            acc8 |= ((t8[w] >> 15) & 0x00010001u) << (2 * w);
            acc4 |= ((t4.u >> 15) & 0x00010001u) << (2 * w);
        }
        mid = (acc8 & 0xffffu) | ((acc8 >> 16) << 1);
        last = (acc4 & 0xffffu) | ((acc4 >> 16) << 1);
    }
    o.lv1 = mid & ~last;
    o.lv2 = ~mid & 0xffffu;
    // union over the heads: OR over the 16 lanes of the lane group (one DPP row)
    u32 both = mid | (last << 16);
    both |= (u32)__builtin_amdgcn_update_dpp(0, (int)both, 0x128, 0xf, 0xf, false);   // row_ror:8
    both |= (u32)__builtin_amdgcn_update_dpp(0, (int)both, 0x124, 0xf, 0xf, false);   // row_ror:4
    both |= (u32)__builtin_amdgcn_update_dpp(0, (int)both, 0x122, 0xf, 0xf, false);   // row_ror:2
    both |= (u32)__builtin_amdgcn_update_dpp(0, (int)both, 0x121, 0xf, 0xf, false);   // row_ror:1
    o.need = both;
}

template <int D, bool REF>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void mfma_v_pass_kernel(
    const uint8_t *__restrict__ first_8, const uint8_t *__restrict__ mid_4, const uint8_t *__restrict__ last_4,
    const unsigned short *__restrict__ probs, const uint8_t *__restrict__ amin_u8, float *__restrict__ partial,
    uint8_t *__restrict__ levels_out, int levels_stride, uint8_t *__restrict__ amin_out, StepGeom geo,
    int tokens_per_wave, int n_chunks, u32 probs_bytes, int max_listed) {
    constexpr int CPP = D / 16;        // channels per lane
    constexpr int MACRO = 64;          // tokens per macro step: 4 tiles of 16 tokens
    __shared__ float fold[4][4][D];    // [wave][head of the pass][channel]
    const int lane = threadIdx.x & 63, wave = wave_index();
    int chunk, hkv, b;
    if (!step_block(geo, chunk, hkv, b)) return;
    const int G = geo.G;
    const int bh_kv = b * geo.Hkv + hkv;
    const int64_t bh0 = (int64_t)b * geo.Hq + hkv * G;
    int n_tokens, nrest;
    seq_state(geo, b, n_tokens, nrest);
    if (chunk * 4 * tokens_per_wave >= n_tokens && chunk > 0) {
        // (without a task map) a workgroup past the end of this sequence only clears its partial sums
        for (int i = threadIdx.x; i < G * D; i += 256) partial[((bh0 + i / D) * n_chunks + chunk) * D + i % D] = 0.f;
        return;
    }
    // all of these are multiples of 64: a step of 16 tokens is inside [t_begin, t_end) or outside as a whole
    const int t_begin = (chunk * 4 + wave) * tokens_per_wave;
    const int t_end = min(t_begin + tokens_per_wave, n_tokens);
    const int64_t row0 = (int64_t)bh_kv * geo.max_seq_len;
    const __amdgpu_buffer_rsrc_t rH = make_rsrc(first_8 + row0 * D, (u32)n_tokens * D);
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(mid_4 + row0 * (D / 2), (u32)n_tokens * (D / 2));
    const __amdgpu_buffer_rsrc_t rL = make_rsrc(last_4 + row0 * (D / 2), (u32)n_tokens * (D / 2));
    const __amdgpu_buffer_rsrc_t rP = make_rsrc(probs, probs_bytes);
    const int j = lane & 15, kq = lane >> 4;
    const bool head = j < G;
    // The threshold is requested here and first looked at behind the requests of the first tiles and probabilities (the
    // barrier below keeps the compiler from waiting for it in front of them: a round trip with nothing else in flight).
    // (a lane without a head reads out of range: zero comes back, and no load sits under a branch)
    const unsigned char amin_loaded =
        (unsigned char)__builtin_amdgcn_raw_buffer_load_b8(make_rsrc(amin_u8 + bh0, (u32)G), (REF || !head) ? kSkip : j, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    const int lane_p = (int)((bh0 + (head ? j : 0)) * geo.row_stride + 4 * kq) * 2;
    const int lane_h = (4 * kq) * D + (lane & 15) * CPP, lane_m = (4 * kq) * (D / 2) + (lane & 15) * (CPP / 2);

    // probabilities of the lane's head for a macro step: 4 steps x 4 tokens (base + 16 s + 4 kq + r)
    auto load_probs = [&](u32x2 *dst, int base) {
        const int o = (base < t_end && head) ? lane_p + base * 2 : kSkip;
#pragma unroll
        for (int sidx = 0; sidx < 4; ++sidx) dst[sidx] = __builtin_amdgcn_raw_buffer_load_b64(rP, o + 32 * sidx, 0, 0);
    };
    // fine(o, s): some lane of the wave fetches a nibble row in step s of the macro step (wave-uniform)
    auto fine = [&](const VMacroOps &o, int sidx) -> bool {
        return __builtin_amdgcn_ballot_w64(((o.need >> (4 * sidx)) & 0x000f000fu) != 0u) != 0ull;
    };
    auto issue = [&](KTaskTile<CPP> &tile, const VMacroOps &o, int macro_base, int sidx) {
        vt_issue<D>(tile, rH, rM, rL, lane_h, lane_m, macro_base + 16 * sidx, macro_base < t_end, fine(o, sidx),
                    (o.need >> (4 * sidx)) & 0xfu, (o.need >> (16 + 4 * sidx)) & 0xfu);
    };
    f32x4 acc[CPP];
#pragma unroll
    for (int i = 0; i < CPP; ++i) acc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    LevelPuts puts;
    puts.pin();
    // what the levels are measured against; lanes without a head read probabilities of zero, for which this value says
    // level 2.  (Worked out where it is first needed, behind the first requests.)
    auto threshold_operand = [&]() -> u16x2 {
        const unsigned short a16 = head ? (unsigned short)((unsigned)amin_loaded << 10) : (unsigned short)0x0800;
        return (u16x2){a16, a16};
    };

    // Few tokens of the wave below level 2 for any head of the group (the usual case: under 1 % of the (token, head)
    // pairs at batch 32, 32 over 8 heads, but 39 % of the 16-token tiles hold one): every tile is multiplied at level 2
    // from its high bytes alone, and the tokens below level 2 -- listed up front from the probabilities -- are
    // gathered into tiles of their own, 16 tokens each, whose rows are fetched at the level the group needs and add
    // value_at_level - value_at_level_2 (kt_correct).  The first such tile is requested before the loop and has
    // arrived when the loop ends.  Many such tokens (flat attention): the loop below, which corrects tile by tile.
    bool handled = false;
    if constexpr (!REF) {
        constexpr int LIST = 256;      // room of a wave's list; max_listed <= LIST pairs take this path
        __shared__ unsigned short fine_tok[4][LIST];    // per wave: token - t_begin | head << 8 | bit 15: read at level 0
        if (tokens_per_wave <= LIST) {
            auto issue_high = [&](KTaskTile<CPP> &tile, int tok) {      // tokens tok .. tok + 15
                const int oh = tok < t_end ? lane_h + tok * D : kSkip;
#pragma unroll
                for (int u = 0; u < 4; ++u) load_bytes<CPP>(tile.h[u], rH, oh + u * D);
            };
            // ---- the list: (token, head) pairs below level 2; every lane notes those of its head ----
            unsigned short *list = fine_tok[wave];
            int n_fine = 0;
            // All probabilities of the group's heads for the wave's tokens in one round trip (they are the operands of the
            // loop below as well), requested in front of the first tiles: loads come back in the order they were issued,
            // and the list waits for the probabilities only.  They come as whole rows -- a request of the wave covers the
            // 256 tokens of two heads, 16 bytes a lane -- and go through LDS into the operand layout (macro step mi, step s,
            // tokens 4 kq + 0..3 of the lane's head): sixteen 8-byte requests per lane, a quarter of the lanes active,
            // cost the pass 7.8 us of 38 at batch 32, 32 over 8 heads, lengths 2048 to 8192.
            constexpr int PS = LIST + 16;       // halves between two heads' rows in LDS (the step keeps the reads off each other's banks)
            __shared__ __attribute__((aligned(16))) unsigned short wave_probs[4][16 * PS];
            unsigned short *wp = wave_probs[wave];
            u32x4 prow[8];
            {
                const int tok = t_begin + (lane & 31) * 8;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int h = 2 * i + (lane >> 5);
                    prow[i] = __builtin_amdgcn_raw_buffer_load_b128(rP, (h < G && tok < t_end) ? (int)((bh0 + h) * geo.row_stride + tok) * 2 : kSkip, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            KTaskTile<CPP> t[4];
#pragma unroll
            for (int i = 0; i < 3; ++i) issue_high(t[i], t_begin + 16 * i);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                *reinterpret_cast<u32x4 *>(wp + (2 * i + (lane >> 5)) * PS + (lane & 31) * 8) = prow[i];
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // the rows are read by other lanes of the wave
            u32x2 pall[LIST / MACRO][4];
#pragma unroll
            for (int mi = 0; mi < LIST / MACRO; ++mi)
#pragma unroll
                for (int sidx = 0; sidx < 4; ++sidx) {
                    const u32x2 v = *reinterpret_cast<const u32x2 *>(wp + (head ? j : 0) * PS + mi * MACRO + 16 * sidx + 4 * kq);
                    pall[mi][sidx] = head ? v : (u32x2){0u, 0u};
                }
            const u16x2 a2 = threshold_operand();
            const unsigned char amin = amin_loaded;
            {
                const i16x2 c8 = {0x0800, 0x0800};
                unsigned long long mask = 0ull;
#pragma unroll
                for (int mi = 0; mi < LIST / MACRO; ++mi) {
                    u32 m16 = 0;
#pragma unroll
                    for (int w = 0; w < 8; ++w) {
                        // 16-bit differences of two tokens (wrapping like the reference's `short` arithmetic,
                        // extension/csrc/V_cache.cu:195-197,211): below level 2 <=> diff < 0x0800
                        union { i16x2 v; u32 u; } x;
                        x.v = __builtin_elementwise_sub_sat(wrap_diff16(a2, (w & 1) ? pall[mi][w >> 1].y : pall[mi][w >> 1].x), c8);
                        m16 |= (((x.u >> 15) & 1u) | ((x.u >> 30) & 2u)) << (2 * w);
                    }
                    mask |= (unsigned long long)m16 << (16 * mi);
                }
                while (__builtin_amdgcn_ballot_w64(mask != 0ull) != 0ull) {
                    const bool on = mask != 0ull;
                    const int bit = on ? __builtin_ctzll(mask) : 0;
                    const int mi = bit >> 4, sidx = (bit >> 2) & 3, u = bit & 3;
                    // the probability itself, for the flag "read at level 0"
                    u32 pb = 0;
#pragma unroll
                    for (int a = 0; a < LIST / MACRO; ++a)
#pragma unroll
                        for (int c = 0; c < 4; ++c)
                            if (a == mi && c == sidx) pb = (u & 2) ? pall[a][c].y : pall[a][c].x;
                    pb = (u & 1) ? pb >> 16 : pb & 0xffffu;
                    const u32 entry = (u32)(64 * mi + 16 * sidx + 4 * kq + u) | ((u32)j << 8) |
                                      ((v_level(amin, (unsigned short)pb) == 0 ? 1u : 0u) << 15);
                    const unsigned long long bm = __builtin_amdgcn_ballot_w64(on);
                    const int at = n_fine + (int)__builtin_amdgcn_mbcnt_hi((u32)(bm >> 32), __builtin_amdgcn_mbcnt_lo((u32)bm, 0u));
                    if (on && at < LIST) list[at] = (unsigned short)entry;
                    n_fine += __builtin_popcountll(bm);
                    mask &= mask - 1ull;
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // the list is read by other lanes of the wave
            if (n_fine <= max_listed) {
                handled = true;
                // ---- a tile of listed pairs: lane group kq takes the entries e0 + 4 kq + u (their rows at the pair's
                //      level; the probability only in the lane of the pair's head, zero for the other heads) ----
                KTaskTile<CPP> ct;
                u32 cp[4];              // probability bits of the lane's head for its group's 4 tokens
                u32 c_mid = 0, c_last = 0;
                auto request_listed = [&](int e0) {
                    c_mid = c_last = 0;
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const int e = e0 + 4 * kq + u;
                        const bool on = e < n_fine;
                        const u32 entry = on ? (u32)list[e] : 0u;
                        const int tok = t_begin + (int)(entry & 0xffu);
                        const bool mine = on && ((entry >> 8) & 15u) == (u32)j;     // the pair's head is this lane's
                        const bool last = on && (entry >> 15) != 0u;
                        load_bytes<CPP>(ct.h[u], rH, on ? tok * D + (lane & 15) * CPP : kSkip);
                        load_bytes<CPP / 2>(ct.m[u], rM, on ? tok * (D / 2) + (lane & 15) * (CPP / 2) : kSkip);
                        load_bytes<CPP / 2>(ct.l[u], rL, last ? tok * (D / 2) + (lane & 15) * (CPP / 2) : kSkip);
                        cp[u] = mine ? (u32)wp[j * PS + (int)(entry & 0xffu)] : 0u;
                        c_mid |= (on ? 1u : 0u) << u;
                        c_last |= (last ? 1u : 0u) << u;
                    }
                };
                auto apply_listed = [&]() {
                    u32 b2[4], b1[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const int lv = v_level(amin, (unsigned short)cp[u]);
                        b2[u] = lv < 2 ? cp[u] : 0u;
                        b1[u] = lv == 1 ? (cp[u] ^ 0x8000u) : 0u;
                    }
                    kt_correct<CPP>(acc, ct, c_mid, c_last, as_f16x4(b1[0] | (b1[1] << 16), b1[2] | (b1[3] << 16)),
                                    as_f16x4(b2[0] | (b2[1] << 16), b2[2] | (b2[3] << 16)), puts);
                };
                request_listed(0);
                __builtin_amdgcn_sched_barrier(0);
                // ---- every tile at level 2 ----
#pragma unroll
                for (int mi = 0; mi < LIST / MACRO; ++mi) {
                    const int base = t_begin + mi * MACRO;
                    if (base < t_end) {
#pragma unroll
                        for (int si = 0; si < 4; ++si) {
                            issue_high(t[(si + 3) & 3], base + 16 * (si + 3));
                            __builtin_amdgcn_sched_barrier(0);
                            kt_compute_coarse<CPP>(acc, t[si], as_f16x4(pall[mi][si].x, pall[mi][si].y));
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
                // ---- the listed tokens: what their levels add to level 2 ----
                for (int e0 = 0; e0 < n_fine; e0 += 16) {
                    if (e0 > 0) request_listed(e0);
                    apply_listed();
                }
            }
        }
    }
    if (!handled) {
    u32x2 pn[4], pnn[4];
    VMacroOps oc, on;
    u16x2 a2;
    {
        u32x2 pc[4];
        load_probs(pc, t_begin);
        load_probs(pn, t_begin + MACRO);
        __builtin_amdgcn_sched_barrier(0);
        a2 = threshold_operand();
        v_macro_ops<REF>(oc, pc, a2, head);
    }
    KTaskTile<CPP> t[4];
#pragma unroll
    for (int i = 0; i < 3; ++i) issue(t[i], oc, t_begin, i);
    __builtin_amdgcn_sched_barrier(0);
    for (int base = t_begin; base < t_end; base += MACRO) {
        load_probs(pnn, base + 2 * MACRO);
        v_macro_ops<REF>(on, pn, a2, head);     // levels and fetch masks of the next macro step
#pragma unroll
        for (int si = 0; si < 4; ++si) {
            if (si == 0) issue(t[3], oc, base, 3);
            else issue(t[si - 1], on, base + MACRO, si - 1);
            __builtin_amdgcn_sched_barrier(0);
            if (fine(oc, si)) {
                const u32 l1 = (oc.lv1 >> (4 * si)) & 0xfu, l2 = (oc.lv2 >> (4 * si)) & 0xfu;
                const u32 pa = oc.p[si].x, pb = oc.p[si].y;
                const u32 m1a = (l1 & 1u ? 0xFFFFu : 0u) | (l1 & 2u ? 0xFFFF0000u : 0u), m1b = (l1 & 4u ? 0xFFFFu : 0u) | (l1 & 8u ? 0xFFFF0000u : 0u);
                const u32 m2a = (l2 & 1u ? 0xFFFFu : 0u) | (l2 & 2u ? 0xFFFF0000u : 0u), m2b = (l2 & 4u ? 0xFFFFu : 0u) | (l2 & 8u ? 0xFFFF0000u : 0u);
                kt_compute<REF, CPP>(acc, t[si], 0, (oc.need >> (4 * si)) & 0xfu, (oc.need >> (16 + 4 * si)) & 0xfu,
                                     as_f16x4(pa & ~(m1a | m2a), pb & ~(m1b | m2b)), as_f16x4(pa & m1a, pb & m1b),
                                     as_f16x4(pa & m2a, pb & m2b), puts);
            } else {
                kt_compute_coarse<CPP>(acc, t[si], as_f16x4(oc.p[si].x, oc.p[si].y));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        oc = on;
#pragma unroll
        for (int i = 0; i < 4; ++i) pn[i] = pnn[i];
    }
    }
    // optional record of the levels, outside the pipeline
    if (!REF && head && amin_out != nullptr && chunk == 0 && wave == 0 && kq == 0) amin_out[bh0 + j] = amin_loaded;
    if (levels_out != nullptr) {
        for (int tt = t_begin + lane; tt < t_end; tt += 64)
            for (int h = 0; h < G; ++h)
                levels_out[(bh0 + h) * levels_stride + tt] =
                    (uint8_t)(REF ? 0 : v_level(amin_u8[bh0 + h], probs[(bh0 + h) * geo.row_stride + tt]));
    }
    // lane (j, ig): acc[cc][r] = out_j[CPP * (4 ig + r) + cc] over this wave's tokens; the 4 waves are added
    // through LDS, four heads at a time
    for (int pass = 0; pass * 4 < G; ++pass) {
        if ((j >> 2) == pass) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int cc = 0; cc < CPP; ++cc) fold[wave][j & 3][CPP * (4 * (lane >> 4) + r) + cc] = acc[cc][r];
        }
        __syncthreads();
        for (int i = threadIdx.x; i < 4 * D; i += 256) {
            const int hs = i / D, d = i - hs * D, hh = pass * 4 + hs;
            if (hh < G)
                partial[((bh0 + hh) * n_chunks + chunk) * D + d] = (fold[0][hs][d] + fold[1][hs][d]) + (fold[2][hs][d] + fold[3][hs][d]);
        }
        __syncthreads();
    }
}

template <int D>
VPlan mfma_v_plan(int B, int Hkv, int n_tokens) {
    VPlan p;
    p.tuned = true;
    // Macro steps of 64 tokens per wave: as many as leave a workgroup for each of the 512 slots (two per compute unit), up
    // to the four whose probabilities a lane keeps in registers.  A workgroup's first 4 to 5 us go by before its stream
    // runs, so fewer and longer ones win: for 256 rows of 1024 / 2048 / 3072 / 4096 / 6144 tokens the pass takes
    // 18.1 / 30.0 / 42.8 / 56.1 / 81.6 us with one step per wave, 15.3 / 21.6 / 30.8 / 39.1 / 56.0 with two and
    // 21.4 / 23.1 / 27.2 / 32.7 / 44.5 with four (above four the pass leaves its fast path: 41.6 us with eight at 4096).
    int k = 1;
    while (k < 4 && (int64_t)B * Hkv * ((n_tokens + 1024 * k - 1) / (1024 * k)) >= 512) k *= 2;
    p.iters_per_wave = k;
    p.tokens_per_wave = 64 * k;
    p.chunk_tokens = 4 * p.tokens_per_wave;
    p.n_chunks = n_tokens > 0 ? (n_tokens + p.chunk_tokens - 1) / p.chunk_tokens : 0;
    return p;
}

template <int D>
int launch_mfma_v_pass(const uint8_t *f8, const uint8_t *m4, const uint8_t *l4, const unsigned short *probs,
                       const uint8_t *amin, float *partial, uint8_t *levels_out, int levels_stride, uint8_t *amin_out,
                       const StepGeom &geo, int B, const VPlan &p, bool ref, hipStream_t st) {
    const int64_t probs_bytes = (int64_t)B * geo.Hq * geo.row_stride * 2;
    if (probs_bytes >= ((int64_t)1 << 31)) {
        set_error("decode_step: probability rows of %lld bytes exceed the 2 GiB the grouped V pass addresses", (long long)probs_bytes);
        return AKV_ERR_INVALID;
    }
    dim3 grid(p.n_chunks, geo.Hkv, B);
    // pairs below level 2 per wave up to which they are listed and corrected in tiles of their own (at most 256: the
    // room of the list; negative: always the loop that corrects tile by tile)
    int max_listed = 48;
    { AKV_TUNE("AKV_TUNE_V_LISTED", v); if (has_v) max_listed = v < 0 ? -1 : (v > 256 ? 256 : v); }
    if (ref)
        hipLaunchKernelGGL((mfma_v_pass_kernel<D, true>), grid, dim3(256), 0, st, f8, m4, l4, probs, amin, partial, levels_out,
                           levels_stride, amin_out, geo, p.tokens_per_wave, p.n_chunks, (u32)probs_bytes, max_listed);
    else
        hipLaunchKernelGGL((mfma_v_pass_kernel<D, false>), grid, dim3(256), 0, st, f8, m4, l4, probs, amin, partial, levels_out,
                           levels_stride, amin_out, geo, p.tokens_per_wave, p.n_chunks, (u32)probs_bytes, max_listed);
    return check_launch("decode_step(mfma v_pass)");
}

#define AKV_INST_K(DD)                                                                                                \
    template int launch_mfma_k_pass<DD>(const uint8_t *, const uint8_t *, const uint8_t *, const uint8_t *,           \
                                        const unsigned short *, const unsigned short *, unsigned short *, uint8_t *, \
                                        u32 *, const StepGeom &, int, int, bool, float, hipStream_t, PassShape *, bool);
#define AKV_INST_V(DD)                                                                                                \
    template VPlan mfma_v_plan<DD>(int, int, int);                                                                    \
    template int launch_mfma_v_pass<DD>(const uint8_t *, const uint8_t *, const uint8_t *, const unsigned short *,    \
                                        const uint8_t *, float *, uint8_t *, int, uint8_t *, const StepGeom &, int,    \
                                        const VPlan &, bool, hipStream_t);
AKV_INST_K(64)
AKV_INST_K(128)
AKV_INST_V(64)
AKV_INST_V(128)   // head_dim 256 keeps the vector-ALU passes: 32-bit level masks, and the V tiles do not fit the registers
#undef AKV_INST_K
#undef AKV_INST_V

}  // namespace akv
