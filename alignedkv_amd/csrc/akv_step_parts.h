// Device-side building blocks of the fused decode step (akv_fused.hip): the K pass over one 256-token stretch of a
// (batch, head) row and the middle stage of a row (append, tail scores, softmax, probe, threshold, tail output).
#pragma once

#include "akv_step.h"

namespace akv {

// K pass over the 256-token stretch `chunk` of a row of planes with 64-token blocks, by a workgroup of four waves: a wave
// takes one block and requests all its rows at once (16 KiB in flight for head_dim 128, no loop).  bh_kv / bh: row of
// the planes (KV head) and of q / the scores (query head).  Scores are stored at device scope.
template <int D, bool REF>
__device__ __forceinline__ void k_pass64_whole_blocks(
    const uint8_t *__restrict__ first_8, const uint8_t *__restrict__ mid_4, const uint8_t *__restrict__ last_4,
    const uint8_t *__restrict__ kcm, const unsigned short *__restrict__ q, const unsigned short *__restrict__ k_new,
    unsigned short *__restrict__ scores, uint8_t *__restrict__ levels_out, const StepGeom &geo, float scale, int chunk, int bh_kv,
    int bh, int R) {
    constexpr int CB = 64;
    constexpr int NG = D / 16;
    static_assert(D <= 128, "a wave holds every channel of a block: head_dim 64 or 128");
    const int lane = threadIdx.x & 63, wave = wave_index();
    const int n_blocks = R / CB;
    const int blk = chunk * 4 + wave;    // may lie past the end: the wave then only helps staging
    const int64_t plane_off = (int64_t)bh_kv * geo.n_max_blocks * (D * (CB / 2));
    // q, the column maxima and the new key of the thread's channel first (loads come back in the order they were issued:
    // behind the plane rows these three would be waited for as long as the rows take), then the block's high bytes.
    static_assert(D <= 256, "a thread stages at most one channel");
    const int sc = threadIdx.x < D ? (int)threadIdx.x : kSkip / 2;
    const u32 s_q = (u32)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(make_rsrc(q + (int64_t)bh * D, D * 2), sc * 2, 0, 0);
    const u32 s_kn = (u32)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(make_rsrc(k_new + (int64_t)bh_kv * D, D * 2), sc * 2, 0, 0);
    const u32 s_cm = (u32)(unsigned char)__builtin_amdgcn_raw_buffer_load_b8(make_rsrc(kcm + (int64_t)bh_kv * D, D), sc, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    KHalfTile<NG> ta;
    k_issue_half_h<D, NG>(ta, make_rsrc(first_8 + plane_off * 2, (u32)n_blocks * (D * CB)), blk, 0);
    __builtin_amdgcn_sched_barrier(0);
    // q and the exponent sums of all channels, staged once per workgroup (three scattered global loads per
    // channel and wave otherwise: half as many load instructions again as the planes themselves need)
    __shared__ u32 staged[D];      // [channel]: q bits | exponent sum << 16
    __shared__ u32 staged_max[4];  // [wave]: largest exponent sum among the channels the wave staged
    {
        // column max including the token appended by this step (a thread without a channel read zeros)
        const u32 cm = max(s_cm, exp_field(s_kn));
        u32 es = threadIdx.x < D ? (exp_field(s_q) + cm) & 0xffu : 0u;
        if (threadIdx.x < D) staged[threadIdx.x] = s_q | (es << 16);
        es = wave_max_u32(es);
        if (lane == 0) staged_max[wave] = es;
    }
    __syncthreads();
    const u32 mx = max(max(staged_max[0], staged_max[1]), max(staged_max[2], staged_max[3]));
    float qf[NG];
    u32 need_mid = 0, need_last = 0;
#pragma unroll
    for (int g = 0; g < NG; ++g) {
        const u32 w = staged[g * 16 + (lane >> 2)];
        qf[g] = lo_half_to_float(w);
        const int lv = REF ? 0 : k_level((unsigned char)mx, (unsigned char)(w >> 16));
        need_mid |= (lv < 2 ? 1u : 0u) << g;
        need_last |= (lv == 0 ? 1u : 0u) << g;
    }
    // (the optional record of the levels: one branch outside the loop, so that the loop's LDS reads go out together)
    if (levels_out != nullptr && chunk == 0 && wave == 0 && (lane & 3) == 0) {
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            const int lv = ((need_last >> g) & 1u) ? 0 : (((need_mid >> g) & 1u) ? 1 : 2);
            levels_out[(int64_t)bh * D + g * 16 + (lane >> 2)] = (uint8_t)lv;
        }
    }
    if (blk < n_blocks)
        k_score_block_whole<D>(ta, mid_4 + plane_off, last_4 + plane_off, n_blocks, blk, qf, need_mid, need_last,
                               scores + (int64_t)bh * geo.row_stride, scale, geo.scores_through != 0);
}

// K pass over one 256-token block `blk` of the (batch, head) row `bh` of planes with 256-token blocks, by a workgroup of
// NWV waves: each wave takes 1/NWV of the channels, requests all its rows at once (12 KiB per wave with four waves and
// head_dim 128) and the partial scores are added through LDS.  R: flushed tokens of the row (the last block may be
// partly filled).  Scores are stored at device scope.
template <int D, bool REF, int NWV>
__device__ __forceinline__ void k_pass256_split_block(
    const uint8_t *__restrict__ first_8, const uint8_t *__restrict__ mid_4, const uint8_t *__restrict__ last_4,
    const uint8_t *__restrict__ kcm, const unsigned short *__restrict__ q, const unsigned short *__restrict__ k_new,
    unsigned short *__restrict__ scores, uint8_t *__restrict__ levels_out, const StepGeom &geo, float scale, int blk, int bh,
    int R) {
    constexpr int KB = 256;
    constexpr int NG = D / 4;      // load groups of 4 channels
    constexpr int HG = 4;          // groups per half tile
    constexpr int GW = NG / NWV;   // groups per wave
    constexpr int NT = GW / HG;    // half tiles per wave
    static_assert(GW % HG == 0 && NG <= 32, "head_dim 64 or 128");
    const int lane = threadIdx.x & 63, wave = wave_index();
    const int n_blocks = (R + KB - 1) / KB;     // the last one may be partly filled
    const int64_t plane_off = (int64_t)bh * geo.n_max_blocks * (D * (KB / 2));
    const __amdgpu_buffer_rsrc_t rH = make_rsrc(first_8 + plane_off * 2, (u32)n_blocks * (D * KB));
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(mid_4 + plane_off, (u32)n_blocks * (D * KB / 2));
    const __amdgpu_buffer_rsrc_t rL = make_rsrc(last_4 + plane_off, (u32)n_blocks * (D * KB / 2));
    const int g_first = wave * GW;
    // q, the column maxima and the new key of the thread's channel first: loads come back in the order they were
    // issued, so behind the plane rows these three would be waited for as long as the rows take, and the nibble rows
    // (which need the levels) would leave a whole round trip after the high bytes instead of right behind them.
    static_assert(D <= 64 * NWV, "a thread stages at most one channel");
    const int sc = threadIdx.x < D ? (int)threadIdx.x : kSkip / 2;
    const u32 s_q = (u32)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(make_rsrc(q + (int64_t)bh * D, D * 2), sc * 2, 0, 0);
    const u32 s_kn = (u32)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(make_rsrc(k_new + (int64_t)bh * D, D * 2), sc * 2, 0, 0);
    const u32 s_cm = (u32)(unsigned char)__builtin_amdgcn_raw_buffer_load_b8(make_rsrc(kcm + (int64_t)bh * D, D), sc, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    KHalfTile<HG> t[NT];
#pragma unroll
    for (int i = 0; i < NT; ++i) k256_issue_h<D, HG>(t[i], rH, blk, g_first + HG * i);
    __builtin_amdgcn_sched_barrier(0);
    __shared__ u32 staged[D];      // [channel]: q bits | exponent sum << 16
    __shared__ u32 staged_max[NWV];  // [wave]: largest exponent sum among the channels the wave staged
    __shared__ float part[NWV][KB];  // [wave][slot]: partial scores
    {
        // column max including the token appended by this step (a thread without a channel read zeros)
        const u32 cm = max(s_cm, exp_field(s_kn));
        u32 es = threadIdx.x < D ? (exp_field(s_q) + cm) & 0xffu : 0u;
        if (threadIdx.x < D) staged[threadIdx.x] = s_q | (es << 16);
        es = wave_max_u32(es);
        if (lane == 0) staged_max[wave] = es;
    }
    __syncthreads();
    u32 mx = 0;
#pragma unroll
    for (int w = 0; w < NWV; ++w) mx = max(mx, staged_max[w]);
    float qf[GW];
    u32 need_mid = 0, need_last = 0;   // bit g: of the wave's group g
#pragma unroll
    for (int g = 0; g < GW; ++g) {
        const u32 w = staged[4 * (g_first + g) + (lane >> 4)];
        qf[g] = lo_half_to_float(w);
        const int lv = REF ? 0 : k_level((unsigned char)mx, (unsigned char)(w >> 16));
        need_mid |= (lv < 2 ? 1u : 0u) << g;
        need_last |= (lv == 0 ? 1u : 0u) << g;
    }
    // (the optional record of the levels: one branch outside the loop, so that the loop's LDS reads go out together)
    if (levels_out != nullptr && blk == 0 && (lane & 15) == 0) {
#pragma unroll
        for (int g = 0; g < GW; ++g) {
            const int lv = ((need_last >> g) & 1u) ? 0 : (((need_mid >> g) & 1u) ? 1 : 2);
            levels_out[(int64_t)bh * D + 4 * (g_first + g) + (lane >> 4)] = (uint8_t)lv;
        }
    }
#pragma unroll
    for (int i = 0; i < NT; ++i)
        k256_issue_ml<D, HG>(t[i], rM, rL, blk, g_first + HG * i, need_mid << g_first, need_last << g_first);
    __builtin_amdgcn_sched_barrier(0);
    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
    for (int i = 0; i < NT; ++i) k_compute_half<HG>(acc, t[i], HG * i, qf, need_mid, need_last);
    reduce_scatter_step<16>(acc, 32);
    reduce_scatter_step<8>(acc, 16);
    const int slot = (lane & 15) * 16 + ((lane & 32) ? 8 : 0) + ((lane & 16) ? 4 : 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) part[wave][slot + i] = acc[i];
    __syncthreads();
    for (int sl = threadIdx.x; sl < KB; sl += 64 * NWV) {
        const int token = blk * KB + sl;
        if (token < R) {
            float sum = 0.f;
#pragma unroll
            for (int w = 0; w < NWV; ++w) sum += part[w][sl];
            // The scores are read by the step's next kernel.  Left in L2 they are written back when the kernel ends, which
            // is cheaper than writing them through while the planes stream as long as they are few: 31.3 instead of 32.0 us
            // for the pass at batch 8 x 32 heads x 4096 tokens (2 MB of scores), but 149.7 instead of 146.0 at 4 x 32 x 32768
            // (8 MB), so the host picks by their volume.
            store_score(make_rsrc(scores + (int64_t)bh * geo.row_stride, (u32)R * 2), token * 2, float_to_half_bits(sum * scale),
                        geo.scores_through != 0);
        }
    }
}

struct MiddleArgs {
    const unsigned short *q, *k_new, *v_new, *mask;
    unsigned short *restk, *restv, *scores, *probs, *otail;
    uint8_t *kcm, *vcm, *toe, *amin;
    const uint8_t *v_first_8;
    StepGeom g;
    int mask_stride;
    int top_k;
    int record_probs;      // 0: the form of the step that keeps the probabilities on chip does not write them to `probs`
    int persist;  // this kernel appends the token (it is not in the rest buffers / planes yet)
};

struct NoHook {
    template <typename I>
    __device__ __forceinline__ void operator()(I) const {}
};
template <int I>
struct HookPoint {
    static constexpr int value = I;
};

// LDS of the middle stage of one (batch, head) row, NW waves.
template <int D, int NW>
struct MiddleShared {
    float red_max[NW], red_sum[NW];    // the waves' row maxima / sums (each written once per stage)
    unsigned short tail_s[64];     // fp16 scores of the tail (mask not yet added)
    float tail_p[64];              // probabilities of the tail
    u32 cand_key[4 * NW][32];      // [16-lane row of the workgroup][residue class]: best (probability, token) key
    float tail_o[NW][D];           // per-wave sums of the tail's share of the output
    u32 vcm[D];                    // V column maxima after the append
    u32 amin;                      // the row's alignment threshold
};

// the tail's share of channel d of the output: the waves' sums in a fixed order
template <int D, int NW>
__device__ __forceinline__ float middle_tail_output(const MiddleShared<D, NW> &ms, int d) {
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) sum += ms.tail_o[w][d];
    return sum;
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding
// global store of the wave (here: 8 KiB of probabilities on their way to memory), which nobody inside the
// middle stage reads back; the stage ends with a full barrier.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// red: written once between two uses of the stage (no barrier needed in front of the write)
template <int NW>
__device__ __forceinline__ float block_reduce(float v, bool is_max, float *red) {
    v = is_max ? wave_max(v) : wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    lds_barrier();
    float r = red[0];
#pragma unroll
    for (int w = 1; w < NW; ++w) r = is_max ? fmaxf(r, red[w]) : r + red[w];
    return r;
}

// Decodes 8 fp16 scores (one 16-byte vector) into floats, adding the fp16 mask in fp16 if there is one.
__device__ __forceinline__ void decode_scores8(const u32x4 w, const unsigned short *mrow, int t0, float *x) {
    const u32 ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const u32 lo = ww[j] & 0xffffu, hi = ww[j] >> 16;
        if (mrow == nullptr) {
            x[2 * j] = half_bits_to_float(lo);
            x[2 * j + 1] = half_bits_to_float(hi);
        } else {
            x[2 * j] = half_bits_to_float(float_to_half_bits(half_bits_to_float(lo) + half_bits_to_float(mrow[t0 + 2 * j])));
            x[2 * j + 1] = half_bits_to_float(float_to_half_bits(half_bits_to_float(hi) + half_bits_to_float(mrow[t0 + 2 * j + 1])));
        }
    }
}

// What a thread of the middle stage keeps for the tail's share of the output (middle_tail_partials): its 16-byte
// pieces of the tail's value rows, requested with the stage's first loads.
template <int D, int NT>
struct MiddleCarry {
    static constexpr int VPR = D / 8;                // 16-byte vectors per row
    static constexpr int NRG = NT / VPR;             // row groups
    static constexpr int MAXR = (64 + NRG - 1) / NRG;
    static_assert(VPR <= 32, "head_dim above 256 needs another tail mapping");
    u32x4 tvw[MAXR];
    int nrest;
};

// The tail's share of the output, an fp16 matmul result (extension/v_cache_file.py:189): a thread takes 8 channels of
// every NRG-th tail token, lanes of a wave that share the channels fold by shuffles; leaves the wave's sums in
// ms.tail_o[wave] (the caller synchronises and adds the waves up: middle_tail_output).  Needs ms.tail_p.
template <int D, int NT>
__device__ __forceinline__ void middle_tail_partials(MiddleShared<D, NT / 64> &ms, const MiddleCarry<D, NT> &c) {
    using C = MiddleCarry<D, NT>;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c8 = tid % C::VPR, rg = tid / C::VPR;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
#pragma unroll
    for (int k = 0; k < C::MAXR; ++k) {
        const int r = rg + k * C::NRG;
        const u32 vv[4] = {c.tvw[k].x, c.tvw[k].y, c.tvw[k].z, c.tvw[k].w};
        const float pr = r < c.nrest ? ms.tail_p[r] : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc[2 * i] = fmaf(lo_half_to_float(vv[i]), pr, acc[2 * i]);
            acc[2 * i + 1] = fmaf(hi_half_to_float(vv[i]), pr, acc[2 * i + 1]);
        }
    }
#pragma unroll
    for (int mk = C::VPR; mk < 64; mk <<= 1)
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] += __shfl_xor(acc[i], mk, 64);
    if (lane < C::VPR) {
#pragma unroll
        for (int i = 0; i < 8; ++i) ms.tail_o[wave][c8 * 8 + i] = acc[i];
    }
}

// The middle stage of one (batch, head) row by the NT threads (a multiple of 256) of one workgroup: append, scores of
// the tail, softmax, probe, threshold, the tail's share of the output.
// hook(HookPoint<i>): a caller that goes on in the same workgroup requests its own data there.  SPLIT = false: i = 0,
// called once the loads that depend on nothing have been requested (loads return in order, so these come back first).
// SPLIT = true: called when the stage's own loads have all arrived (i = 0; requests made earlier share the memory
// system with the stage's first loads and hold them back by as long as they take themselves: measured 4 us for 16 KiB
// per wave), after the row maximum (1), after the row sum (2) and when the probabilities are out (3): a wave cannot
// run ahead of a load the compute unit's memory pipeline has no room for yet, so what is to travel during the stage
// is requested piece by piece between its phases.
// probs_lds (may be null): LDS copy of the row's probabilities, tokens 0 .. R + tail, for a caller that goes on in the
// same workgroup.
// SPLIT = false: the whole stage; threshold in a.amin (and ms.amin), tail output in a.otail.
// SPLIT = true (needs R > 0): everything up to the probabilities, the residue classes' candidates (ms.cand_key), the
// column maxima (ms.vcm) and the tail's probabilities (ms.tail_p), ending with an LDS barrier; the caller lets one wave
// run middle_probe_wave (probe and threshold, no barrier inside) while the others go on, and calls
// middle_tail_partials with `carry` when it suits it (every wave, before the workgroup adds up ms.tail_o).
// MASKED: 1 / 0 = the caller knows that there is / is no mask row (the other case is not compiled), -1 = looked up at
// run time.  MAXTOK: an upper bound of the flushed tokens per row that the caller guarantees (0: none; rows beyond
// what the registers hold take three passes over the scores): both keep a one-shot kernel's code short.
template <int D, int NW, typename Waiting>
__device__ __forceinline__ u32 middle_probe_wave(const MiddleArgs &a, MiddleShared<D, NW> &ms, int bh, int R, Waiting while_waiting);

template <int D, int NT, bool SPLIT = false, typename Hook = NoHook, int MASKED = -1, int MAXTOK = 0>
__device__ __forceinline__ void middle_body(const MiddleArgs &a, const int bh, MiddleShared<D, NT / 64> &ms, Hook hook = Hook(),
                                            unsigned short *probs_lds = nullptr, MiddleCarry<D, NT> *carry_out = nullptr) {
    // 16-byte score vectors a thread keeps in registers
    constexpr int VPT = MAXTOK > 0 ? (MAXTOK / 8 + NT - 1) / NT : 4;
    constexpr int NW = NT / 64;               // waves
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // bh indexes (batch, query head); the keys, values, column maxima and rest buffers belong to its KV head
    const int b = bh / a.g.Hq, hq = bh - b * a.g.Hq, h = hq / a.g.G;
    const int bh_kv = b * a.g.Hkv + h;
    const int Hkv = a.g.Hkv, cb = a.g.cb;
    const bool owner = hq % a.g.G == 0;       // one query head of the group writes the shared state
    int R, nrest;
    seq_state<SPLIT>(a.g, b, R, nrest);      // (SPLIT: the one-launch second half of the step, uniform lengths only)
    const int newest = nrest - 1;
    const unsigned short *qrow = a.q + (int64_t)bh * D;
    const unsigned short *knew = a.k_new + (int64_t)bh_kv * D;
    const unsigned short *vnew = a.v_new + (int64_t)bh_kv * D;
    unsigned short *srow = a.scores + (int64_t)bh * a.g.row_stride;
    unsigned short *prow = a.probs + (int64_t)bh * a.g.row_stride;
    const unsigned short *mrow = MASKED == 0 ? nullptr : ((MASKED == 1 || a.mask) ? a.mask + (int64_t)b * a.mask_stride : nullptr);
    const int nvec = R >> 3;
    const bool in_regs = MAXTOK > 0 || nvec <= NT * VPT;
    // scores of the flushed part are read at device scope: other workgroups of the same launch wrote them
    const __amdgpu_buffer_rsrc_t rScores = make_rsrc(srow, (u32)R * 2);
    // (SPLIT: the caller reads the probabilities from LDS; their copy in memory is a record for the host)
    const bool to_memory = !SPLIT || a.record_probs != 0;
    auto store_probs8 = [&](int i, const u32x4 o) {
        if (probs_lds != nullptr) *reinterpret_cast<u32x4 *>(probs_lds + i * 8) = o;
        if (to_memory) *reinterpret_cast<u32x4 *>(prow + i * 8) = o;
    };
    auto store_prob1 = [&](int t, unsigned short p) {
        if (probs_lds != nullptr) probs_lds[t] = p;
        if (to_memory) prow[t] = p;
    };

    // Everything that does not depend on anything else is requested first: the score vectors of the
    // flushed part, the new token, the column maxima and the tail's key and value rows.
    u32x4 sv[VPT];
    if (in_regs) {
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            const int i = tid + NT * v;
            sv[v] = load_b128_device(rScores, i < nvec ? i * 16 : kSkip);
        }
    }
    // the tail's key rows and q: LPT lanes per tail token, 8 channels per 16-byte load, all rows in flight at once
    // (a real decode step has 32 tail tokens on average)
    constexpr int LPT = NT / 64;              // lanes per token (the rest buffer holds at most 64 tokens)
    constexpr int NKV = (D / 8 + LPT - 1) / LPT;
    const int tr = tid / LPT, tj = tid % LPT;
    u32x4 tkw[NKV], tqw[NKV];
    // All of these are buffer loads whose offset is out of range where a lane has nothing to fetch (zeros come back):
    // no load sits under a branch, so the compiler issues them back to back and the stage starts with one round trip.
    // Rest buffers of this (batch, KV head): row r at r * Hkv * D; the newest token comes from k_new / v_new while
    // this kernel is the one that appends it.
    const u32 rest_bytes = (u32)(((cb - 1) * Hkv + 1) * D * 2);
    const __amdgpu_buffer_rsrc_t rRK = make_rsrc(a.restk + ((int64_t)b * cb * Hkv + h) * D, rest_bytes);
    const __amdgpu_buffer_rsrc_t rRV = make_rsrc(a.restv + ((int64_t)b * cb * Hkv + h) * D, rest_bytes);
    const __amdgpu_buffer_rsrc_t rQ = make_rsrc(qrow, D * 2), rKN = make_rsrc(knew, D * 2), rVN = make_rsrc(vnew, D * 2);
    const bool fresh = a.persist != 0;
    {
#pragma unroll
        for (int i = 0; i < NKV; ++i) {
            const int v8 = tj + i * LPT;
            const bool on = tr < nrest && v8 < D / 8, is_new = fresh && tr == newest;
            const u32x4 kr = __builtin_amdgcn_raw_buffer_load_b128(rRK, (on && !is_new) ? (tr * Hkv * D + v8 * 8) * 2 : kSkip, 0, 0);
            const u32x4 kn = __builtin_amdgcn_raw_buffer_load_b128(rKN, (on && is_new) ? v8 * 16 : kSkip, 0, 0);
            tkw[i] = kr | kn;
            tqw[i] = __builtin_amdgcn_raw_buffer_load_b128(rQ, on ? v8 * 16 : kSkip, 0, 0);
        }
    }
    // value rows of the tail, used by (f): a thread takes 8 channels of every NRG-th tail token
    using Carry = MiddleCarry<D, NT>;
    Carry carry;
    carry.nrest = nrest;
    auto request_tail_values = [&]() {
        const int c8 = tid % Carry::VPR, rg = tid / Carry::VPR;
#pragma unroll
        for (int k = 0; k < Carry::MAXR; ++k) {
            const int r = rg + k * Carry::NRG;
            const bool on = r < nrest, is_new = fresh && r == newest;
            const u32x4 vr = __builtin_amdgcn_raw_buffer_load_b128(rRV, (on && !is_new) ? (r * Hkv * D + c8 * 8) * 2 : kSkip, 0, 0);
            const u32x4 vn = __builtin_amdgcn_raw_buffer_load_b128(rVN, (on && is_new) ? c8 * 16 : kSkip, 0, 0);
            carry.tvw[k] = vr | vn;
        }
    };
    // (SPLIT: with the first loads, so that nothing the stage needs later queues behind the caller's stream)
    if (SPLIT) request_tail_values();
    // (a) append the token: rest buffers and column maxima (extension/k_cache_file.py:98-101).
    static_assert(D <= NT, "one channel per thread");
    const bool ch_on = tid < D;               // this thread looks after channel tid of the column maxima
    const int ch = ch_on ? tid : 0;
    u32 kc = (u32)(unsigned char)__builtin_amdgcn_raw_buffer_load_b8(make_rsrc(a.kcm + (int64_t)bh_kv * D, D), ch_on ? ch : kSkip, 0, 0);
    u32 vc = (u32)(unsigned char)__builtin_amdgcn_raw_buffer_load_b8(make_rsrc(a.vcm + (int64_t)bh_kv * D, D), ch_on ? ch : kSkip, 0, 0);
    const u32 kb = (u32)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(rKN, ch_on ? ch * 2 : kSkip, 0, 0);
    const u32 vb = (u32)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(rVN, ch_on ? ch * 2 : kSkip, 0, 0);
    if constexpr (!SPLIT) {
        __builtin_amdgcn_sched_barrier(0);
        hook(HookPoint<0>());
        __builtin_amdgcn_sched_barrier(0);
    }
    // Every query head of the group derives the updated maxima itself (max is idempotent, so it does not matter
    // whether it reads them before or after the owner's store, nor whether an earlier kernel of the step has
    // appended the token already).
    kc = max(kc, exp_field(kb));
    vc = max(vc, exp_field(vb));
    if (ch_on) ms.vcm[ch] = vc;
    // The stores of the append: issued here, where the wave waits for its first loads anyway, and in front of the
    // tail's score store -- a wait for a loaded value placed behind a store would also wait for that store to be
    // acknowledged (one counter covers both), a round trip in front of the stage's first barrier.
    if (a.persist && owner && ch_on) {
        const int64_t at = (((int64_t)b * cb + newest) * Hkv + h) * D + ch;
        a.restk[at] = (unsigned short)kb;
        a.restv[at] = (unsigned short)vb;
        a.kcm[(int64_t)bh_kv * D + ch] = (uint8_t)kc;
        a.vcm[(int64_t)bh_kv * D + ch] = (uint8_t)vc;
    }
    // (b) scores of the tail: fp16(fp16(q.k) / sqrt(D)), the two roundings of an fp16 matmul followed by
    //     an fp16 division (extension/k_cache_file.py:156)
    const float sqrt_d = sqrtf((float)D);
    {
        float part = 0.f;
#pragma unroll
        for (int i = 0; i < NKV; ++i) {
            const u32 kk[4] = {tkw[i].x, tkw[i].y, tkw[i].z, tkw[i].w}, qq[4] = {tqw[i].x, tqw[i].y, tqw[i].z, tqw[i].w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                part = fmaf(lo_half_to_float(kk[c]), lo_half_to_float(qq[c]), part);
                part = fmaf(hi_half_to_float(kk[c]), hi_half_to_float(qq[c]), part);
            }
        }
        part = lane_group_sum<LPT>(part);
        if (tr < nrest && tj == 0) {
            const float dot16 = half_bits_to_float(float_to_half_bits(part));
            const unsigned short sc = float_to_half_bits(dot16 / sqrt_d);
            ms.tail_s[tr] = sc;
            srow[R + tr] = sc;
        }
    }
    lds_barrier();
    // SPLIT: the stage's loads are all back; from here to the probe it only computes, and memory is the caller's
    auto hook_at = [&](auto point) {
        if constexpr (SPLIT) {
            __builtin_amdgcn_sched_barrier(0);
            hook(point);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    hook_at(HookPoint<0>());

    // (c) softmax over [0, R + nrest): scores + mask in fp16, softmax in fp32, probabilities in fp16
    //     (model/KVCache_AlignedKV.py:119-121), and the running arg-max of the residue classes mod 32:
    //     vector i holds tokens 8i..8i+7, a thread's vectors are 256 apart, so its j-th token always has
    //     residue (8*(tid&3) + j) mod 32.
    auto masked1 = [&](u32 sbits, int t) -> float {
        if (mrow == nullptr) return half_bits_to_float(sbits);
        return half_bits_to_float(float_to_half_bits(half_bits_to_float(sbits) + half_bits_to_float(mrow[t])));
    };
    // arg-max key of a token: probability bits (fp16 of a non-negative number: ordered like an integer)
    // in the high half, 0xFFFF - (token / 32) in the low half: the largest key is the largest probability
    // and, among equals, the smallest token (first maximal index, as torch.max returns it)
    u32 best[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) best[j] = 0u;
    const float xt = tid < nrest ? masked1(ms.tail_s[tid], R + tid) : -INFINITY;
    float m = xt, sum = 0.f;
    auto emit_probs8 = [&](int i, const float *e, float rsum) {
        u32 out[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const u32 p0 = float_to_half_bits(div_by(e[2 * j], sum, rsum)), p1 = float_to_half_bits(div_by(e[2 * j + 1], sum, rsum));
            out[j] = p0 | (p1 << 16);
            const u32 grp = 0xffffu - (u32)(i >> 2);     // token / 32 = vector index / 4
            best[2 * j] = max(best[2 * j], (p0 << 16) | grp);
            best[2 * j + 1] = max(best[2 * j + 1], (p1 << 16) | grp);
        }
        const u32x4 o = {out[0], out[1], out[2], out[3]};
        store_probs8(i, o);
    };
    if (in_regs) {
        float x[VPT][8];
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            const int i = tid + NT * v;
            if (i < nvec) {
                decode_scores8(sv[v], mrow, i * 8, x[v]);
#pragma unroll
                for (int j = 0; j < 8; ++j) m = fmaxf(m, x[v][j]);
            }
        }
        m = block_reduce<NW>(m, true, ms.red_max);
        hook_at(HookPoint<1>());
#pragma unroll
        for (int v = 0; v < VPT; ++v)
            if (tid + NT * v < nvec) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    x[v][j] = exp_nonpositive(x[v][j] - m);
                    sum += x[v][j];
                }
            }
        const float et = tid < nrest ? exp_nonpositive(xt - m) : 0.f;
        sum = block_reduce<NW>(sum + et, false, ms.red_sum);
        hook_at(HookPoint<2>());
        const float rsum = 1.0f / sum;
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            const int i = tid + NT * v;
            if (i < nvec) emit_probs8(i, x[v], rsum);
        }
        if (tid < nrest) {
            const unsigned short p = float_to_half_bits(div_by(et, sum, rsum));
            store_prob1(R + tid, p);
            ms.tail_p[tid] = half_bits_to_float(p);
        }
    } else {
        // long rows: three passes over the scores (they stay in the L2 of this workgroup's XCD)
        float x[8];
        for (int i = tid; i < nvec; i += NT) {
            decode_scores8(load_b128_device(rScores, i * 16), mrow, i * 8, x);
#pragma unroll
            for (int j = 0; j < 8; ++j) m = fmaxf(m, x[j]);
        }
        m = block_reduce<NW>(m, true, ms.red_max);
        for (int i = tid; i < nvec; i += NT) {
            decode_scores8(load_b128_device(rScores, i * 16), mrow, i * 8, x);
#pragma unroll
            for (int j = 0; j < 8; ++j) sum += exp_nonpositive(x[j] - m);
        }
        const float et = tid < nrest ? exp_nonpositive(xt - m) : 0.f;
        sum = block_reduce<NW>(sum + et, false, ms.red_sum);
        const float rsum = 1.0f / sum;
        hook_at(HookPoint<1>());
        hook_at(HookPoint<2>());
        for (int i = tid; i < nvec; i += NT) {
            decode_scores8(load_b128_device(rScores, i * 16), mrow, i * 8, x);
#pragma unroll
            for (int j = 0; j < 8; ++j) x[j] = exp_nonpositive(x[j] - m);
            emit_probs8(i, x, rsum);
        }
        if (tid < nrest) {
            const unsigned short p = float_to_half_bits(div_by(et, sum, rsum));
            store_prob1(R + tid, p);
            ms.tail_p[tid] = half_bits_to_float(p);
        }
    }

    hook_at(HookPoint<3>());
    // value rows of the tail: requested here so that they travel while the probe runs
    if (!SPLIT) request_tail_values();

    // (d) candidates of the probe over the flushed part (extension/v_cache_file.py:119-143): thread tid saw residues
    //     8*(tid&3)+j.  Lanes of a 16-lane row that share (tid&3): two row rotations (DPP); then one LDS row per
    //     16-lane row (the arg-max over these rows is taken by whoever runs the probe).
    if (R > 0) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            best[j] = max(best[j], (u32)__builtin_amdgcn_update_dpp(0, (int)best[j], 0x124, 0xf, 0xf, false));   // row_ror:4
            best[j] = max(best[j], (u32)__builtin_amdgcn_update_dpp(0, (int)best[j], 0x128, 0xf, 0xf, false));   // row_ror:8
        }
        if ((lane & 15) < 4) {
#pragma unroll
            for (int j = 0; j < 8; ++j) ms.cand_key[tid >> 4][8 * (lane & 3) + j] = best[j];
        }
    }
    lds_barrier();
    // (e) the probe's arg-max per residue class, its 32 gathered rows and the alignment threshold of this (batch, head)
    //     (extension/v_cache_file.py:156-160)
    if constexpr (!SPLIT) {
        // one wave runs the probe (no barrier inside); the others go on to the tail's share of the output
        if (R > 0 && wave == 0) middle_probe_wave<D, NW>(a, ms, bh, R, [] {});
    }
    // (f) the tail's share of the output
    if constexpr (SPLIT) {
        *carry_out = carry;
    } else {
        middle_tail_partials<D, NT>(ms, carry);
        lds_barrier();
        for (int d = tid; d < D; d += NT) a.otail[(int64_t)bh * D + d] = float_to_half_bits(middle_tail_output<D, NW>(ms, d));
    }
}

// The probe and the alignment threshold of a row by ONE wave (no workgroup barrier inside), after middle_body<SPLIT>:
// the arg-max of every residue class from the waves' candidates, the 32 gathered high-byte rows (lane = D / 64
// neighbouring channels, a row per load instruction, the row's token in a scalar register), the probe's exponents and
// the threshold, which goes to a.amin and ms.amin.  extension/v_cache_file.py:119-143,156-160.
// while_waiting: called once the gather has been requested.
template <int D, int NW, typename Waiting>
__device__ __forceinline__ u32 middle_probe_wave(const MiddleArgs &a, MiddleShared<D, NW> &ms, int bh, int R, Waiting while_waiting) {
    constexpr int CPL = D / 64;               // channels per lane
    static_assert(CPL == 1 || CPL == 2 || CPL == 4, "head_dim 64, 128 or 256");
    const int lane = threadIdx.x & 63;
    const int b = bh / a.g.Hq, hq = bh - b * a.g.Hq, h = hq / a.g.G;
    const int bh_kv = b * a.g.Hkv + h;
    // arg-max of residue class r = lane % 32 over the candidates of half of the rows; the two halves meet in scalar
    // registers below
    const int r = lane & 31, half = lane >> 5;
    u32 key = 0u;
#pragma unroll
    for (int k = 0; k < 2 * NW; ++k) key = max(key, ms.cand_key[half * 2 * NW + k][r]);
    const __amdgpu_buffer_rsrc_t rF = make_rsrc(a.v_first_8 + (int64_t)bh_kv * a.g.max_seq_len * D, (u32)R * D);
    u32 hi[32], pbits[32];
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const u32 k_i = max((u32)__builtin_amdgcn_readlane((int)key, i), (u32)__builtin_amdgcn_readlane((int)key, i + 32));
        pbits[i] = k_i >> 16;
        const int row = ((int)(0xffffu - (k_i & 0xffffu)) * 32 + i) * D;
        if constexpr (CPL == 1) hi[i] = (u32)(unsigned char)__builtin_amdgcn_raw_buffer_load_b8(rF, lane, row, 0);
        else if constexpr (CPL == 2) hi[i] = (u32)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(rF, lane * 2, row, 0);
        else hi[i] = __builtin_amdgcn_raw_buffer_load_b32(rF, lane * 4, row, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    while_waiting();
    __builtin_amdgcn_sched_barrier(0);
    float acc[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) acc[c] = 0.f;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const float p = half_bits_to_float(pbits[i]);
#pragma unroll
        for (int c = 0; c < CPL; ++c)
            acc[c] = fmaf(half_bits_to_float(((((hi[i] >> (8 * c)) & 0xffu) << 8) | 0x80u) & 0x7fffu), p, acc[c]);
    }
    u32 align = 0xffu;
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
        // exponent with the lowest bit cleared (`& 0x1F - 1`, extension/v_cache_file.py:142)
        const u32 e = exp_field(float_to_half_bits(acc[c])) & 0x1eu;
        a.toe[(int64_t)bh * D + lane * CPL + c] = (uint8_t)e;
        align = min(align, (e + 15u - ms.vcm[lane * CPL + c]) & 0xffu);     // uint8 wrap, as the reference's tensor arithmetic
    }
    align = wave_min_u32(align);
    if (lane == 0) {
        a.amin[bh] = (uint8_t)align;
        ms.amin = align;
    }
    return align;
}

}  // namespace akv
