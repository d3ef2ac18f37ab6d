// Fused AlignedKV decode step: append one token per sequence and attend over the whole cache in
// four launches (K pass, middle, V pass, combine) instead of the reference's three custom launches
// plus ~25 small framework kernels per layer (reference: model/KVCache_AlignedKV.py:101-124,
// extension/k_cache_file.py:97-118,132-159, extension/v_cache_file.py:97-116,119-190).
//
//   K pass   scores of the flushed blocks; the fetch level of every channel is derived in the
//            kernel from q, the column-max exponents and the new key (k_cache_file.py:98-99,136-138)
//   middle   one workgroup per (batch, head): appends the token to the fp16 rest buffers and
//            updates the column maxima, scores of the unflushed tail, mask, fp32 softmax -> fp16
//            probabilities, arg-max of every residue class mod top_max_k, the output-magnitude
//            probe, and the tail's share of the output
//   V pass   split over the sequence; the alignment threshold of the (batch, head) is derived in
//            the kernel from the probe exponents and the V column maxima (v_cache_file.py:156-160)
//   combine  adds the chunk partials in a fixed order, rounds to fp16 and adds the fp16 tail part
// On a step that fills the rest buffer (64 tokens) a persist kernel and the two plane-write kernels
// run first, exactly as the reference flushes before it computes.
#include "akv_step_parts.h"

#include <mutex>

namespace akv {

// defined in akv_k.hip / akv_v.hip
int launch_k_save_blocks(uint8_t *first_8, uint8_t *mid_4, uint8_t *last_4, const uint8_t *k_new, int bsz, int heads,
                         int n_blocks, int n_max_blocks, int d_head, int d_block, int start_pos, int seqlen,
                         hipStream_t st);
int launch_v_save(uint8_t *first_8, uint8_t *mid_4, uint8_t *last_4, const uint8_t *v_new, int bsz, int heads,
                  int max_seq_len, int head_dim, int start_pos, int seq_len, int v_new_seq, hipStream_t st);

// Optional per-phase timing of the fused step (benchmark aid): when enabled, events are recorded on the
// step's stream around the K pass, the middle kernel, the V pass and the combine kernel.  Process-wide and
// unsynchronised on purpose: for a single-threaded benchmark that runs one step at a time on one stream.
static bool g_profile = false;
static hipEvent_t g_ev[7];   // 0..4 around the four phases, 5 and 6 back to back (interval of an empty phase)
static bool g_ev_ready = false;
static inline void mark(int i, hipStream_t st) {
    if (g_profile) (void)hipEventRecord(g_ev[i], st);
}


// ------------------------------------------------------------------------------------------------
// persist (flush steps only): token -> rest buffers, column maxima.  grid (B*H), D threads.
// ------------------------------------------------------------------------------------------------
__global__ void fused_persist_kernel(const unsigned short *__restrict__ k_new, const unsigned short *__restrict__ v_new,
                                     unsigned short *__restrict__ restk, unsigned short *__restrict__ restv,
                                     uint8_t *__restrict__ kcm, uint8_t *__restrict__ vcm, int H, int D, int cb, int slot) {
    const int bh = blockIdx.x, b = bh / H, h = bh - b * H;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        u32 kb = k_new[(int64_t)bh * D + d], vb = v_new[(int64_t)bh * D + d];
        int64_t at = (((int64_t)b * cb + slot) * H + h) * D + d;
        restk[at] = (unsigned short)kb;
        restv[at] = (unsigned short)vb;
        kcm[(int64_t)bh * D + d] = (uint8_t)max((u32)kcm[(int64_t)bh * D + d], exp_field(kb));
        vcm[(int64_t)bh * D + d] = (uint8_t)max((u32)vcm[(int64_t)bh * D + d], exp_field(vb));
    }
}

// Task maps of a step with per-sequence lengths (see step_block): for each of the two streaming passes the
// workgroups that have tokens to read, ordered by (batch, head index, chunk) with the chunk fastest, then kNoTask
// up to the size of the grid; v_chunks[b] = V-pass chunks of sequence b, for the combine kernel (the lengths
// themselves advance while it runs).  One workgroup of 256 threads per sequence and map: it sums the entry counts
// of the sequences before its own, writes its sequence's entries and its share of the kNoTask tail.
struct TaskMaps {
    u32x2 *map_k, *map_v;    // null: no map for that pass
    int *v_chunks;
    PassShape k, v;
};

__device__ __forceinline__ void build_task_map(const StepGeom &geo, u32x2 *map, const PassShape &sh, int B, int *v_chunks,
                                               int *red, int b_mine) {
    const int tid = threadIdx.x;
    auto chunks_of = [&](int b) {
        int R, nrest;
        seq_state(geo, b, R, nrest);
        // (never more than the grid holds, whatever the length says: the map has grid_x entries per head)
        return min((R + sh.tokens_per_wg - 1) / sh.tokens_per_wg, sh.grid_x);
    };
    int before = 0, all = 0;
    for (int b = tid; b < B; b += 256) {
        const int c = chunks_of(b) * sh.grid_y;
        all += c;
        if (b < b_mine) before += c;
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        before += __shfl_xor(before, m, 64);
        all += __shfl_xor(all, m, 64);
    }
    if ((tid & 63) == 0) {
        red[2 * (tid >> 6)] = before;
        red[2 * (tid >> 6) + 1] = all;
    }
    __syncthreads();
    const int at = red[0] + red[2] + red[4] + red[6], total = red[1] + red[3] + red[5] + red[7];
    const int n = chunks_of(b_mine), cnt = n * sh.grid_y;
    if (v_chunks != nullptr && tid == 0) v_chunks[b_mine] = n;
    const u32 len_mine = (u32)geo.seq_lens[b_mine];
    for (int i = tid; i < cnt; i += 256) {
        const int y = i / n, x = i - y * n;
        map[at + i] = u32x2{pack_task(x, y, b_mine), len_mine};
    }
    // the entries past the last task: an equal share per workgroup
    const int grid = sh.grid_x * sh.grid_y * B, tail = grid - total, share = (tail + B - 1) / B;
    for (int i = b_mine * share + tid; i < min((b_mine + 1) * share, tail); i += 256) map[total + i] = u32x2{kNoTask, 0u};
}

// extra = index among the 2 * B map workgroups: the first B build the K pass's map, the others the V pass's
__device__ __forceinline__ void build_task_maps(const StepGeom &geo, const TaskMaps &m, int B, int *red, int extra) {
    if (extra < B) {
        if (m.map_k != nullptr) build_task_map(geo, m.map_k, m.k, B, nullptr, red, extra);
    } else {
        if (m.map_v != nullptr) build_task_map(geo, m.map_v, m.v, B, m.v_chunks, red, extra - B);
    }
}

// Ragged mode, first kernel of every step: append the token of every sequence to its rest buffer, update the
// column maxima and, for the sequences whose rest buffer is full with it, write the 64-token block into the
// planes (same bytes as k_save_blocks_kernel / v_save_vec8_kernel).  kPreSplit workgroups per (batch, KV head):
// the first appends, and a flush is shared between them (16 tokens of V and a quarter of the channels of K each;
// the token of this step is taken from the step's inputs, so no workgroup waits for the append).
// grid (B*Hkv*kPreSplit [+ ceil(B*Hkv/4) for the set-up of the matrix-core K pass] [+ 2*B for the task maps]), 256 threads.
constexpr int kPreSplit = 4;
// what the matrix-core K pass wants set up per (batch, KV head) (mfma_k_prepare); words == nullptr: nothing
struct KPrepare {
    const unsigned short *q;
    u32 *words;
    uint8_t *levels_out;
    int ref;
};
template <int D>
__global__ __launch_bounds__(256) void fused_pre_kernel(uint8_t *__restrict__ kf8, uint8_t *__restrict__ km4,
                                                        uint8_t *__restrict__ kl4, uint8_t *__restrict__ vf8,
                                                        uint8_t *__restrict__ vm4, uint8_t *__restrict__ vl4,
                                                        const unsigned short *__restrict__ k_new,
                                                        const unsigned short *__restrict__ v_new,
                                                        unsigned short *__restrict__ restk, unsigned short *__restrict__ restv,
                                                        uint8_t *__restrict__ kcm, uint8_t *__restrict__ vcm, StepGeom geo,
                                                        TaskMaps maps, int B, KPrepare prep) {
    constexpr int CB = 64, S = kPreSplit, DS = D / S, TS = CB / S;
    static_assert(DS % 8 == 0, "a workgroup's share of the channels is a whole number of 16-byte vectors");
    __shared__ unsigned short tile[CB][DS + 2];
    __shared__ int map_scratch[8];
    const int n_bh = B * geo.Hkv;
    const int n_prep = prep.words != nullptr ? (n_bh + 3) / 4 : 0;
    if ((int)blockIdx.x >= n_bh * S + n_prep) {   // the last workgroups: task maps of the K pass and of the V pass
        build_task_maps(geo, maps, B, map_scratch, (int)blockIdx.x - n_bh * S - n_prep);
        return;
    }
    if ((int)blockIdx.x >= n_bh * S) {   // set-up of the matrix-core K pass, a wave per (batch, KV head)
        if constexpr (D <= 128) {
            const int bh_kv = ((int)blockIdx.x - n_bh * S) * 4 + wave_index();
            if (bh_kv < n_bh) {
                if (prep.ref) mfma_k_prepare<D, true>(kcm, prep.q, k_new, prep.words, prep.levels_out, geo, bh_kv);
                else mfma_k_prepare<D, false>(kcm, prep.q, k_new, prep.words, prep.levels_out, geo, bh_kv);
            }
        }
        return;
    }
    const int bh = blockIdx.x / S, sub = blockIdx.x - bh * S, b = bh / geo.Hkv, h = bh - b * geo.Hkv;
    const int cur = geo.seq_lens[b];
    const int slot = cur % CB;
    if (sub == 0) {
        for (int d = threadIdx.x; d < D; d += 256) {
            const u32 kb = k_new[(int64_t)bh * D + d], vb = v_new[(int64_t)bh * D + d];
            const int64_t at = (((int64_t)b * CB + slot) * geo.Hkv + h) * D + d;
            restk[at] = (unsigned short)kb;
            restv[at] = (unsigned short)vb;
            kcm[(int64_t)bh * D + d] = (uint8_t)max((u32)kcm[(int64_t)bh * D + d], exp_field(kb));
            vcm[(int64_t)bh * D + d] = (uint8_t)max((u32)vcm[(int64_t)bh * D + d], exp_field(vb));
        }
    }
    if (slot != CB - 1) return;
    const int blk = cur / CB;
    // row j of the block: the rest buffer, or this step's token for the last one
    auto k_row = [&](int j) { return j == CB - 1 ? k_new + (int64_t)bh * D : restk + (((int64_t)b * CB + j) * geo.Hkv + h) * D; };
    auto v_row = [&](int j) { return j == CB - 1 ? v_new + (int64_t)bh * D : restv + (((int64_t)b * CB + j) * geo.Hkv + h) * D; };
    // V rows sub*TS .. sub*TS + TS - 1: 8 channels per thread and token
    for (int idx = threadIdx.x; idx < TS * (D / 8); idx += 256) {
        const int j = sub * TS + idx / (D / 8), d8 = idx % (D / 8);
        const u32x4 w = *reinterpret_cast<const u32x4 *>(v_row(j) + d8 * 8);
        const u32 ww[4] = {w.x, w.y, w.z, w.w};
        u32 hi0 = 0, hi1 = 0, mid = 0, last = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const u32 e = ww[i] & 0xffffu, o = ww[i] >> 16;
            const u32 hp = (e >> 8) | ((o >> 8) << 8);
            if (i < 2) hi0 |= hp << (16 * i); else hi1 |= hp << (16 * (i - 2));
            mid |= ((e & 0xf0u) | ((o & 0xf0u) >> 4)) << (8 * i);
            last |= (((e & 0x0fu) << 4) | (o & 0x0fu)) << (8 * i);
        }
        const int64_t row = (int64_t)bh * geo.max_seq_len + (int64_t)blk * CB + j;
        const u32x2 hv = {hi0, hi1};
        *reinterpret_cast<u32x2 *>(vf8 + row * D + d8 * 8) = hv;
        *reinterpret_cast<u32 *>(vm4 + row * (D / 2) + d8 * 4) = mid;
        *reinterpret_cast<u32 *>(vl4 + row * (D / 2) + d8 * 4) = last;
    }
    // K block, channels sub*DS .. sub*DS + DS - 1: transpose through LDS
    const int d0 = sub * DS;
    for (int idx = threadIdx.x; idx < CB * (DS / 8); idx += 256) {
        const int j = idx / (DS / 8), d8 = idx % (DS / 8);
        const u32x4 w = *reinterpret_cast<const u32x4 *>(k_row(j) + d0 + d8 * 8);
        const u32 ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            tile[j][d8 * 8 + 2 * i] = (unsigned short)(ww[i] & 0xffffu);
            tile[j][d8 * 8 + 2 * i + 1] = (unsigned short)(ww[i] >> 16);
        }
    }
    __syncthreads();
    // the 64 tokens go to slots s0 .. s0 + 63 of K plane block kblk (blocks of geo.kb tokens)
    const int KB = geo.kb, kblk = (blk * CB) / KB, s0 = blk * CB - kblk * KB;
    const int64_t base = ((int64_t)bh * geo.n_max_blocks + kblk) * (int64_t)D * (KB / 2);
    for (int idx = threadIdx.x; idx < DS * (CB / 4); idx += 256) {
        const int dl = idx / (CB / 4), d = d0 + dl, j = (idx % (CB / 4)) * 4;
        const u32 w = (u32)(tile[j][dl] >> 8) | ((u32)(tile[j + 1][dl] >> 8) << 8) | ((u32)(tile[j + 2][dl] >> 8) << 16) |
                      ((u32)(tile[j + 3][dl] >> 8) << 24);
        *reinterpret_cast<u32 *>(kf8 + base * 2 + (int64_t)d * KB + s0 + j) = w;
    }
    for (int idx = threadIdx.x; idx < DS * (CB / 8); idx += 256) {
        const int dl = idx / (CB / 8), d = d0 + dl, j = (idx % (CB / 8)) * 8;
        u32 mw = 0, lw = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const u32 le = tile[j + 2 * i][dl] & 0xffu, lo = tile[j + 2 * i + 1][dl] & 0xffu;
            mw |= ((le & 0xf0u) | (lo >> 4)) << (8 * i);
            lw |= (((le & 0x0fu) << 4) | (lo & 0x0fu)) << (8 * i);
        }
        *reinterpret_cast<u32 *>(km4 + base + (int64_t)d * (KB / 2) + ((s0 + j) >> 1)) = mw;
        *reinterpret_cast<u32 *>(kl4 + base + (int64_t)d * (KB / 2) + ((s0 + j) >> 1)) = lw;
    }
}


// ------------------------------------------------------------------------------------------------
// K pass.  grid (ceil(n_blocks / (4*blocks_per_wave)), H, B), 256 threads.
// ------------------------------------------------------------------------------------------------
template <int D, bool REF, bool WHOLE = false, bool UNIFORM = false>
__global__ __launch_bounds__(256) void fused_k_pass_kernel(
    const uint8_t *__restrict__ first_8, const uint8_t *__restrict__ mid_4, const uint8_t *__restrict__ last_4,
    const uint8_t *__restrict__ kcm, const unsigned short *__restrict__ q, const unsigned short *__restrict__ k_new,
    unsigned short *__restrict__ scores, uint8_t *__restrict__ levels_out, StepGeom geo, int blocks_per_wave,
    float scale) {
    constexpr int CB = 64;
    constexpr int NG = D / 16;
    const int lane = threadIdx.x & 63, wave = wave_index();
    if constexpr (UNIFORM) fetch_arguments_now(first_8, mid_4, last_4, kcm, q, k_new, scores, levels_out);
    // UNIFORM: one query head per KV head and one length for every sequence (nothing to look up before the first requests)
    int bx = blockIdx.x, hkv = blockIdx.y, b = blockIdx.z, chunk = bx, gq = 0;
    if constexpr (!UNIFORM) {
        if (!step_block(geo, bx, hkv, b)) return;
        decode_group_block(geo.G, bx, chunk, gq);
    }
    const int bh_kv = b * geo.Hkv + hkv, bh = b * geo.Hq + hkv * geo.G + gq;
    int R, nrest;
    seq_state<UNIFORM>(geo, b, R, nrest);
    if constexpr (WHOLE) {
        // blocks_per_wave == 1: every channel of the wave's block is requested at once
        if constexpr (D <= 128) k_pass64_whole_blocks<D, REF>(first_8, mid_4, last_4, kcm, q, k_new, scores, levels_out, geo, scale, chunk, bh_kv, bh, R);
        return;
    }
    const int n_blocks = R / CB;
    const int first_blk = (chunk * 4 + wave) * blocks_per_wave;   // may lie past the end: the wave then idles
    const int end_blk = min(first_blk + blocks_per_wave, n_blocks);

    const int64_t plane_off = (int64_t)bh_kv * geo.n_max_blocks * (D * (CB / 2));
    KHalfTile<D / 32> ta;
    k_prefetch_first<D>(ta, first_8 + plane_off * 2, n_blocks, first_blk);
    // q and the exponent sums of all channels, staged once per workgroup (three scattered global loads per
    // channel and wave otherwise: half as many load instructions again as the planes themselves need)
    __shared__ u32 staged[D];      // [channel]: q bits | exponent sum << 16
    for (int c = threadIdx.x; c < D; c += 256) {
        const u32 qb = q[(int64_t)bh * D + c];
        // column max including the token appended by this step
        const u32 cm = max((u32)kcm[(int64_t)bh_kv * D + c], exp_field(k_new[(int64_t)bh_kv * D + c]));
        staged[c] = qb | (((exp_field(qb) + cm) & 0xffu) << 16);
    }
    __syncthreads();
    float qf[NG];
    u32 esum[NG];
    u32 mx = 0;
#pragma unroll
    for (int g = 0; g < NG; ++g) {
        const u32 w = staged[g * 16 + (lane >> 2)];
        qf[g] = lo_half_to_float(w);
        esum[g] = w >> 16;
        mx = max(mx, esum[g]);
    }
    mx = quads_max_u32(mx);
    u32 need_mid = 0, need_last = 0;
#pragma unroll
    for (int g = 0; g < NG; ++g) {
        const int lv = REF ? 0 : k_level((unsigned char)mx, (unsigned char)esum[g]);
        need_mid |= (lv < 2 ? 1u : 0u) << g;
        need_last |= (lv == 0 ? 1u : 0u) << g;
        if (levels_out != nullptr && chunk == 0 && wave == 0 && (lane & 3) == 0)
            levels_out[(int64_t)bh * D + g * 16 + (lane >> 2)] = (uint8_t)lv;
    }
    k_score_blocks<D>(ta, first_8 + plane_off * 2, mid_4 + plane_off, last_4 + plane_off, n_blocks, first_blk, end_blk, qf,
                      need_mid, need_last, scores + (int64_t)bh * geo.row_stride, scale, 1, geo.scores_through != 0);
}

// K pass over planes with 256-token blocks (multi-head): one workgroup per block, its four waves take a quarter of the
// channels each, request all their rows at once (12 KiB per wave, five waves per SIMD) and add their partial scores
// through LDS.  (A block per wave with double-buffered half tiles measured behind on every shape: 33.9 vs 33.6 us at
// batch 8 x 4096 tokens, 155.2 vs 146.9 at 4 x 32768, 8.1 vs 5.2 at 1 x 1024.)  grid (n_kblocks, H, B), 256 threads.
// UNIFORM: one length for every sequence (no task map and no per-sequence lengths to look up in front of a workgroup's
// first requests).
template <int D, bool REF, int NWV, bool UNIFORM>
__global__ __launch_bounds__(64 * NWV) void fused_k_pass256_split_kernel(
    const uint8_t *__restrict__ first_8, const uint8_t *__restrict__ mid_4, const uint8_t *__restrict__ last_4,
    const uint8_t *__restrict__ kcm, const unsigned short *__restrict__ q, const unsigned short *__restrict__ k_new,
    unsigned short *__restrict__ scores, uint8_t *__restrict__ levels_out, StepGeom geo, float scale) {
    if constexpr (UNIFORM) fetch_arguments_now(first_8, mid_4, last_4, kcm, q, k_new, scores, levels_out);
    int blk = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    if constexpr (!UNIFORM) {
        if (!step_block(geo, blk, h, b)) return;
    }
    int R, nrest;
    seq_state<UNIFORM>(geo, b, R, nrest);
    if (blk >= (R + 255) / 256) return;
    k_pass256_split_block<D, REF, NWV>(first_8, mid_4, last_4, kcm, q, k_new, scores, levels_out, geo, scale, blk, b * geo.Hq + h, R);
}

// ------------------------------------------------------------------------------------------------
// middle.  grid (B*H), 256 threads.
// ------------------------------------------------------------------------------------------------
// grid (B*H), 256 threads: the middle stage on its own (no flushed block yet, or fusion switched off).
template <int D, int NT>
__global__ __launch_bounds__(NT) void fused_middle_kernel(MiddleArgs a) {
    __shared__ MiddleShared<D, NT / 64> ms;
    // Workgroups go to the 8 XCDs round-robin by index.  The G query heads of a KV head read the same rest-buffer rows
    // and probe the same value rows: with indices 8 apart they meet in one XCD's L2.
    int bh = blockIdx.x;
    const int G = a.g.G, n_groups = (int)gridDim.x / G;
    if (G > 1 && (n_groups & 7) == 0) {
        const int t = bh >> 3;
        bh = ((t / G) * 8 + (bh & 7)) * G + t % G;
    }
    middle_body<D, NT>(a, bh, ms);
}

constexpr int tail_rows_per_cu = 2, tail_max_tokens = 8192;


// Second half of a step in one launch: the middle stage, the V pass and the final sum for one (batch, head) per
// workgroup of 8 waves, after a K pass that ran as a launch of its own.  With about as many (batch, head) pairs as
// compute units (or a multiple of them) every unit streams one row of V planes from start to end: no partial sums,
// no combine launch, and the first high-byte tiles of every wave travel while the middle stage runs.
//
// The V planes start to stream as soon as the row's probabilities are known: one wave works out the probe and the
// row's alignment threshold (a gather of 32 rows: a memory round trip of its own) while the other waves multiply
// their first `fa` half tiles each at level 2, which needs no threshold.  After a barrier every wave lists the tokens
// of its share that are below level 2 (from the probabilities in LDS), requests the first of them, streams the rest
// of its share at level 2 and then adds p * (value at the token's level - value at level 2) for the listed tokens.
// A wave whose tokens are below level 2 more often than one in 16 (flat attention) lists only the ones it has
// multiplied already and takes the nibble rows of the others along with their half tiles (v_stream_run).
// grid (B*H), NT threads.
template <int D, int NT, int PRE, bool MASKED>
__global__ __launch_bounds__(NT) void tail_step_kernel(const uint8_t *__restrict__ v_first_8,
                                                        const uint8_t *__restrict__ v_mid_4,
                                                        const uint8_t *__restrict__ v_last_4, MiddleArgs ma,
                                                        unsigned short *__restrict__ out,
                                                        uint8_t *__restrict__ v_levels_out,
                                                        uint8_t *__restrict__ amin_out, int fa) {
    constexpr int NW = NT / 64;
    using S = VStream<D>;
    __shared__ MiddleShared<D, NW> ms;
    __shared__ float wave_part[NW][D];
    // the row's probabilities stay in LDS for the V part (the copy in memory is the step's debug output)
    // (+ 64 zeros behind the row and its tail, for half tiles past a wave's share: see v_stream_run_coarse)
    constexpr int zero_at = tail_max_tokens + 64;
    __shared__ __attribute__((aligned(16))) unsigned short probs_lds[tail_max_tokens + 64 + 64];
    if (threadIdx.x < 64) probs_lds[zero_at + threadIdx.x] = 0;
    __shared__ u32 fine_list[NW][tail_max_tokens / NW];
    fetch_arguments_now(v_first_8, v_mid_4, v_last_4, ma.q, ma.k_new, ma.v_new, ma.mask, ma.restk, ma.restv, ma.scores, ma.probs,
                        ma.kcm, ma.vcm, ma.toe, ma.amin, ma.v_first_8, out, v_levels_out, amin_out, ma.g.row_stride, ma.persist);
    const int wave = wave_index();
    const int bh = blockIdx.x;
    int R, nrest_unused;
    seq_state<true>(ma.g, 0, R, nrest_unused);
    const int64_t row0 = (int64_t)bh * ma.g.max_seq_len;
    const uint8_t *f8 = v_first_8 + row0 * D, *m4 = v_mid_4 + row0 * (D / 2), *l4 = v_last_4 + row0 * (D / 2);
    const __amdgpu_buffer_rsrc_t rH = make_rsrc(f8, (u32)R * D);
    // Part A, before the threshold is known: the first n_a half tiles of the row, dealt out to the waves 1 .. NW - 1
    // (wave 0 runs the probe meanwhile); part B: the others, dealt out to all waves.
    const int n_halves = (R + S::HT - 1) / S::HT;
    const int n_a = min(fa * (NW - 1), n_halves);
    VSeq seq_a, seq_b;
    seq_a.n_halves = seq_b.n_halves = n_halves;
    seq_a.start = wave - 1; seq_a.stride = NW - 1;
    seq_a.count = (wave >= 1 && wave - 1 < n_a) ? (n_a - (wave - 1) + NW - 2) / (NW - 1) : 0;
    seq_b.start = n_a + wave; seq_b.stride = NW;
    seq_b.count = n_a + wave < n_halves ? (n_halves - n_a - wave + NW - 1) / NW : 0;
    // Requested before the middle stage, right behind its first loads, and held in registers until the probabilities
    // are known: the first PRE half tiles of the wave's part A, and the half tile it streams first afterwards.  (The
    // waves 1 .. NW - 1 have no other loads between the stage's first ones and the stream, so nothing of theirs queues
    // behind these; wave 0 has the probe's gather to come and requests only its first half tile of part B.)
    VHighPart<S::HV> pre[PRE > 0 ? PRE : 1];
    VRing<D, 2> ring;
    VSeq seq_a2 = seq_a;        // part A beyond the PRE half tiles held in registers
    seq_a2.start = seq_a.start + PRE * seq_a.stride;
    seq_a2.count = max(seq_a.count - PRE, 0);
    const int first_streamed = wave == 0 ? seq_b.half(0) : (seq_a2.count > 0 ? seq_a2.half(0) : seq_b.half(0));
    MiddleCarry<D, NT> carry;
    static_assert(PRE <= 3, "one half tile per phase of the middle stage");
    auto between_phases = [&](auto point) {
        constexpr int i = decltype(point)::value;
        if constexpr (i < PRE) {
            if (wave != 0) v_stream_issue_high<D>(pre[i], rH, seq_a.half(i));
        }
        if constexpr (i == 3) v_stream_issue_high<D>(ring.hi[0], rH, first_streamed);
    };
    middle_body<D, NT, true, decltype(between_phases), MASKED ? 1 : 0, tail_max_tokens>(ma, bh, ms, between_phases, probs_lds, &carry);
    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    // the tail's share of the output: once per wave, where it hides behind memory time
    bool tail_done = false;
    auto tail_once = [&]() {
        if (!tail_done) middle_tail_partials<D, NT>(ms, carry);
        tail_done = true;
    };
    if (wave == 0) {
        middle_probe_wave<D, NW>(ma, ms, bh, R, tail_once);
    } else {
        const int tl = (threadIdx.x & 63) / S::LPR;
#pragma unroll
        for (int k = 0; k < PRE; ++k) {
            const int half = seq_a.half(k);
            const bool on = half < n_halves;
            u32 sb[S::HV];
#pragma unroll
            for (int u = 0; u < S::HV; ++u) sb[u] = (u32)probs_lds[(on ? half * S::HT : zero_at) + tl + u * S::TPL];
            v_compute_half_coarse<S::HV>(acc, pre[k], sb);
        }
        pin_accumulators(acc);
        // (ends with part B's first half tile requested, unless it was the one requested up front)
        v_stream_run_coarse<D>(ring, f8, R, probs_lds, zero_at, seq_a2, true, seq_b.half(0), acc, [&](int) { tail_once(); });
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    const unsigned char amin = (unsigned char)ms.amin;
    if (amin_out != nullptr && threadIdx.x == 0) amin_out[bh] = amin;
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(m4, (u32)R * (D / 2)), rL = make_rsrc(l4, (u32)R * (D / 2));
    u32 *list = fine_list[wave];
    int count = 0;
    const int n_fine = v_stream_count_fine<D, true>(probs_lds, R, amin, seq_a) + v_stream_count_fine<D, true>(probs_lds, R, amin, seq_b);
    const bool few = n_fine * 16 <= (seq_a.count + seq_b.count) * S::HT;
    VFineScan<D> scan;
    scan.probs_lds = probs_lds; scan.amin = amin; scan.a = seq_a; scan.b = seq_b;
    if (!few) scan.b.count = 0;     // (the others are read at their level as they stream)
    typename VListed<D>::Step first;
    int listed_from = 0;      // `first` holds the list's entries from here on
    if (few) {
        // Part B in two stretches: during the first the tokens below level 2 are listed, 64 tokens per half tile of the
        // stream; then they are requested, and arrive while the second stretch streams.
        const int n_b1 = min(seq_b.count, 2 * ((scan.steps_left() + 1) / 2));
        VSeq b1 = seq_b, b2 = seq_b;
        b1.count = n_b1;
        b2.start = seq_b.start + n_b1 * seq_b.stride; b2.count = seq_b.count - n_b1;
        v_stream_run_coarse<D>(ring, f8, R, probs_lds, zero_at, b1, true, b2.half(0), acc, [&](int) {
            tail_once();
            if (!scan.done()) scan.step(list, count);
        });
        while (!scan.done()) scan.step(list, count);
        VListed<D>::request(first, list, count, 0, rH, rM, rL, amin, 0);
        __builtin_amdgcn_sched_barrier(0);
        v_stream_run_coarse<D>(ring, f8, R, probs_lds, zero_at, b2, true, n_halves, acc);
    } else {
        // Frequent tokens below level 2 (flat attention): the rest of the row streams at the tokens' own levels, and the
        // corrections of what part A multiplied at level 2 ride along, one batch of listed rows per half tile.
        while (!scan.done()) scan.step(list, count);
        VListed<D>::request(first, list, count, 0, rH, rM, rL, amin, 0);
        __builtin_amdgcn_sched_barrier(0);
        v_stream_run_levels<D, 2>(f8, m4, l4, R, probs_lds, zero_at, amin, seq_b, acc, [&](int) {
            VListed<D>::apply(acc, first);
            listed_from += VListed<D>::TPL;
            VListed<D>::request(first, list, count, listed_from, rH, rM, rL, amin, 0);
        });
    }
    tail_once();
    VListed<D>::apply_all(acc, first, list, count, rH, rM, rL, amin, 0, listed_from);
    if (v_levels_out != nullptr)
        for (int t = threadIdx.x; t < R; t += NT) v_levels_out[(int64_t)bh * R + t] = (uint8_t)v_level(amin, probs_lds[t]);
    v_fold_lanes<D, NW>(acc, wave_part);
    __syncthreads();
    for (int d = threadIdx.x; d < D; d += NT) {
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) sum += wave_part[w][d];
        const float o16 = half_bits_to_float(float_to_half_bits(sum));
        // fp16(planes) + fp16(tail), the fp16 `o += tail` of the reference (extension/v_cache_file.py:189)
        const float t16 = half_bits_to_float(float_to_half_bits(middle_tail_output<D, NW>(ms, d)));
        out[(int64_t)bh * D + d] = float_to_half_bits(o16 + t16);
    }
}

// The same for the mode that reads every plane (the reference's `reference=True`): no fetch levels, so the whole
// middle stage runs first and every wave then streams its share with the nibble rows (ring of NR half tiles, the
// first PF of them requested before the middle stage).  grid (B*H), NT threads.
template <int D, int NR, int PF, int NT>
__global__ __launch_bounds__(NT) void tail_step_ref_kernel(const uint8_t *__restrict__ v_first_8,
                                                            const uint8_t *__restrict__ v_mid_4,
                                                            const uint8_t *__restrict__ v_last_4, MiddleArgs ma,
                                                            unsigned short *__restrict__ out,
                                                            uint8_t *__restrict__ v_levels_out) {
    constexpr int NW = NT / 64;
    __shared__ MiddleShared<D, NW> ms;
    __shared__ float wave_part[NW][D];
    const int wave = wave_index();
    const int bh = blockIdx.x;
    int R, nrest_unused;
    seq_state(ma.g, bh / ma.g.Hq, R, nrest_unused);
    const int64_t row0 = (int64_t)bh * ma.g.max_seq_len;
    const uint8_t *f8 = v_first_8 + row0 * D, *m4 = v_mid_4 + row0 * (D / 2), *l4 = v_last_4 + row0 * (D / 2);
    // wave w takes the half tiles w, w + NW, ...
    VSeq seq;
    seq.n_halves = (R + VStream<D>::HT - 1) / VStream<D>::HT;
    seq.start = wave; seq.stride = NW;
    seq.count = wave < seq.n_halves ? (seq.n_halves - wave + NW - 1) / NW : 0;
    VRing<D, NR> ring;
    middle_body<D, NT, false>(ma, bh, ms, [&](auto) { v_stream_prefetch<D, NR, PF>(ring, f8, R, seq); });
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    const unsigned short *prow = ma.probs + (int64_t)bh * ma.g.row_stride;
    v_stream_run<D, true, NR, PF>(ring, f8, m4, l4, R, prow, 0, seq, acc);
    if (v_levels_out != nullptr)
        for (int t = threadIdx.x; t < R; t += NT) v_levels_out[(int64_t)bh * R + t] = 0;
    v_fold_lanes<D, NW>(acc, wave_part);
    __syncthreads();
    for (int d = threadIdx.x; d < D; d += NT) {
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) sum += wave_part[w][d];
        const float o16 = half_bits_to_float(float_to_half_bits(sum));
        out[(int64_t)bh * D + d] = float_to_half_bits(o16 + half_bits_to_float(ma.otail[(int64_t)bh * D + d]));
    }
}

// Threshold indexing of the reference expression as written (extension/v_cache_file.py:157-160): entry b*H+h
// pairs the probe of (b / H, b % H) with the column maxima of (b / H, h).  grid (B*H), 64 threads.
__global__ void fused_amin_literal_kernel(const uint8_t *__restrict__ toe, const uint8_t *__restrict__ vcm,
                                          uint8_t *__restrict__ amin, int H, int D) {
    const int bh = blockIdx.x, b = bh / H, h = bh - b * H;
    const int probe_bh = (b / H) * H + (b % H), cm_bh = (b / H) * H + h;
    u32 mn = 0xffu;
    for (int c = threadIdx.x; c < D; c += 64)
        mn = min(mn, ((u32)toe[(int64_t)probe_bh * D + c] + 15u - (u32)vcm[(int64_t)cm_bh * D + c]) & 0xffu);
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) mn = min(mn, (u32)__shfl_xor((int)mn, m, 64));
    if (threadIdx.x == 0) amin[bh] = (uint8_t)mn;
}

// ------------------------------------------------------------------------------------------------
// V pass.  grid (n_chunks, H, B), 256 threads.
// ------------------------------------------------------------------------------------------------
// UNIFORM: one query head per KV head and one length for every sequence (nothing to look up before the first requests)
template <int D, bool REF, int NIT, bool UNIFORM = false>
__global__ __launch_bounds__(256) void fused_v_pass_kernel(
    const uint8_t *__restrict__ first_8, const uint8_t *__restrict__ mid_4, const uint8_t *__restrict__ last_4,
    const unsigned short *__restrict__ probs, const uint8_t *__restrict__ amin_u8, float *__restrict__ partial,
    uint8_t *__restrict__ levels_out, int levels_stride, uint8_t *__restrict__ amin_out, StepGeom geo,
    int tokens_per_wave, int n_chunks) {
    if constexpr (UNIFORM) fetch_arguments_now(first_8, mid_4, last_4, probs, amin_u8, partial, levels_out, amin_out);
    __shared__ float wave_part[4][D];
    const int wave = wave_index();
    int bx = blockIdx.x, hkv = blockIdx.y, b = blockIdx.z, chunk = bx, gq = 0;
    if constexpr (!UNIFORM) {
        if (!step_block(geo, bx, hkv, b)) return;
        decode_group_block(geo.G, bx, chunk, gq);
    }
    const int bh_kv = b * geo.Hkv + hkv, bh = b * geo.Hq + hkv * geo.G + gq;
    if (chunk >= n_chunks) return;    // padding of the grid (whole workgroup)
    int n_tokens, nrest;
    seq_state<UNIFORM>(geo, b, n_tokens, nrest);
    const int t_begin = (chunk * 4 + wave) * tokens_per_wave;
    const int t_end = min(t_begin + tokens_per_wave, n_tokens);
    const int64_t row0 = (int64_t)bh_kv * geo.max_seq_len;
    // the threshold and (inside v_accumulate) the probabilities before the first rows: the levels wait for them only
    const unsigned char amin = REF ? 0 : amin_u8[bh];
    VFirstTile<D> ft;
    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    v_accumulate<D, REF, NIT, 0, false, true>(ft, first_8 + row0 * D, mid_4 + row0 * (D / 2), last_4 + row0 * (D / 2), n_tokens,
                                        probs + (int64_t)bh * geo.row_stride, amin, t_begin, t_end, acc,
                                        levels_out != nullptr ? levels_out + (int64_t)bh * levels_stride : nullptr);
    if (!REF && amin_out != nullptr && chunk == 0 && threadIdx.x == 0) amin_out[bh] = amin;
    v_fold_workgroup<D>(acc, wave_part, partial + ((int64_t)bh * n_chunks + chunk) * D);
}

// grid (B*H), D threads: out = fp16(fp16(sum of partials) + tail), the fp16 `o += tail` of the reference.
__global__ void fused_combine_kernel(const float *__restrict__ partial, const unsigned short *__restrict__ otail,
                                     unsigned short *__restrict__ out, int D, int n_chunks, int *seq_lens_rw, int Hq,
                                     const int *__restrict__ v_chunks) {
    const int bh = blockIdx.x;
    // with a task map only the chunks of this sequence were written
    const int n_sum = v_chunks != nullptr ? v_chunks[bh / Hq] : n_chunks;
    // last kernel of the step: the sequence lengths kept on the device advance here
    if (seq_lens_rw != nullptr && threadIdx.x == 0 && bh % Hq == 0) seq_lens_rw[bh / Hq] += 1;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        // fixed order (the bits do not depend on which workgroup finished first), eight loads in flight at a time
        const float *src = partial + (int64_t)bh * n_chunks * D + d;
        float acc = 0.f;
        int c = 0;
        for (; c + 8 <= n_sum; c += 8) {
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = src[(int64_t)(c + i) * D];
#pragma unroll
            for (int i = 0; i < 8; ++i) acc += v[i];
        }
        for (; c < n_sum; ++c) acc += src[(int64_t)c * D];
        const float o16 = half_bits_to_float(float_to_half_bits(acc));
        out[(int64_t)bh * D + d] = float_to_half_bits(o16 + half_bits_to_float(otail[(int64_t)bh * D + d]));
    }
}

struct StepLayout {
    size_t toe, amin, otail, partial, prep, map_k, map_v, v_chunks, total;
};

static StepLayout step_layout(int B, int H, int D, int max_seq_len) {
    StepLayout l;
    auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
    const VPlan p = v_plan(B, H, D, max_seq_len);
    // the plan for fewer tokens never has more chunks than the plan for max_seq_len has at its finest split
    size_t max_chunks = (size_t)(max_seq_len + 4 * (D == 256 ? 32 : 64) - 1) / (4 * (D == 256 ? 32 : 64));
    (void)p;
    l.toe = 0;
    l.amin = up((size_t)B * H * D);
    l.otail = l.amin + up((size_t)B * H);
    l.partial = l.otail + up((size_t)B * H * D * 2);
    l.prep = l.partial + up((size_t)B * H * max_chunks * D * sizeof(float));
    l.map_k = l.prep + up((size_t)B * H * mfma_k_prep_words(D) * sizeof(u32));   // B * Hkv <= B * H rows are used
    // task maps: a pass has at most B * H * (max_chunks + 1) workgroups
    l.map_v = l.map_k + up((size_t)B * H * (max_chunks + 1) * sizeof(u32x2));
    l.v_chunks = l.map_v + up((size_t)B * H * (max_chunks + 1) * sizeof(u32x2));
    l.total = l.v_chunks + up((size_t)B * sizeof(int));
    return l;
}

template <int D>
static int run_step(uint8_t *kf8, uint8_t *km4, uint8_t *kl4, uint8_t *vf8, uint8_t *vm4, uint8_t *vl4, uint8_t *kcm,
                    uint8_t *vcm, uint8_t *restk, uint8_t *restv, const uint8_t *q, const uint8_t *k_new,
                    const uint8_t *v_new, const uint8_t *mask, int mask_stride, uint8_t *out, uint8_t *scores,
                    uint8_t *probs, int row_stride, uint8_t *ws, uint8_t *k_levels_out, uint8_t *v_levels_out,
                    uint8_t *amin_out, int B, int Hq, int Hkv, int n_max_blocks, int max_seq_len, int cb, int kb, int top_k,
                    int cur_len, int *seq_lens, bool ref, int flags, hipStream_t st) {
    const int literal_broadcast = flags & AKV_STEP_LITERAL_BROADCAST;
    const StepLayout lay = step_layout(B, Hq, D, max_seq_len);
    uint8_t *toe = ws + lay.toe;
    uint8_t *amin = ws + lay.amin;
    unsigned short *otail = reinterpret_cast<unsigned short *>(ws + lay.otail);
    float *partial = reinterpret_cast<float *>(ws + lay.partial);
    const unsigned short *q16 = reinterpret_cast<const unsigned short *>(q);
    const unsigned short *k16 = reinterpret_cast<const unsigned short *>(k_new);
    const unsigned short *v16 = reinterpret_cast<const unsigned short *>(v_new);
    unsigned short *s16 = reinterpret_cast<unsigned short *>(scores);
    unsigned short *p16 = reinterpret_cast<unsigned short *>(probs);
    unsigned short *rk16 = reinterpret_cast<unsigned short *>(restk), *rv16 = reinterpret_cast<unsigned short *>(restv);
    const bool ragged = seq_lens != nullptr;

    StepGeom geo;
    geo.Hq = Hq; geo.Hkv = Hkv; geo.G = Hq / Hkv;
    geo.cb = cb; geo.max_seq_len = max_seq_len; geo.n_max_blocks = n_max_blocks; geo.row_stride = row_stride;
    geo.kb = kb;
    geo.cur_len = cur_len; geo.seq_lens = seq_lens;
    geo.task_map = nullptr;
    geo.scores_through = (int64_t)B * Hq * (cur_len + 1) * 2 > ((int64_t)4 << 20) ? 1 : 0;

    // flushed tokens after the append: exact for uniform lengths, an upper bound for ragged ones
    const int R = (cur_len + 1) / cb * cb;
    const int n_blocks = R / cb;
    // the kernel multiplies by the fp16-rounded scale (extension/csrc/K_cache.cu:306)
    const float scale = __half2float(__float2half_rn(1.0f / sqrtf((float)D)));
    // grouped-query heads: one workgroup per plane chunk serves 2 or 4 query heads (group_heads),
    // or up to 16 on the matrix cores (K pass)
    const bool grouped = group_heads(geo.G) > 1;
    const bool matrix = geo.G >= 2 && geo.G <= 16 && D <= 128;   // (the 32-bit level masks hold 128 channels)
    if (kb != 64 && geo.G > 1 && !matrix) {
        set_error("decode_step: grouped-query heads over K plane blocks of %d tokens need the matrix-core K pass", kb);
        return AKV_ERR_INVALID;
    }
    const int n_kblocks = (R + kb - 1) / kb;    // K plane blocks that hold tokens (the last one may be partly filled)
    // 64-token K blocks (head_dim 64 and 128): a block per wave with all its rows requested at once; against two blocks
    // per wave in half tiles: 36.8 vs 37.3 us at batch 8 x 4096 tokens, 160.2 vs 163.6 at 4 x 32768
    const bool k_whole = kb == 64 && D <= 128 && !grouped && !matrix;
    const int bpw = (kb == 256 || k_whole) ? 1 : k_blocks_per_wave(B, Hq, n_blocks);
    const bool matrix_v = matrix;
    VPlan p = v_plan(B, grouped ? Hq / group_heads(geo.G) : Hq, D, R);
    if constexpr (D <= 128) {
        if (matrix_v) p = mfma_v_plan<D>(B, Hkv, R);
    }
    // launch shapes of the two streaming passes
    PassShape ks = {0, 0, 0}, vs = {0, 0, 0};
    if (n_blocks > 0) {
        if (matrix) {
            int rc = AKV_OK;
            if constexpr (D <= 128)
                rc = launch_mfma_k_pass<D>(kf8, km4, kl4, kcm, q16, k16, s16, k_levels_out, nullptr, geo, B, n_blocks, ref, scale, st, &ks);
            if (rc != AKV_OK) return rc;
        } else if (grouped) {
            int rc = launch_group_k_pass<D>(kf8, km4, kl4, kcm, q16, k16, s16, k_levels_out, geo, B, n_blocks, ref, scale, st, &ks);
            if (rc != AKV_OK) return rc;
        } else {
            if (kb == 256) ks = PassShape{n_kblocks, Hkv, kb};
            else ks = PassShape{group_grid_x((n_blocks + 4 * bpw - 1) / (4 * bpw), geo.G), Hkv, 4 * bpw * kb};
        }
        if (matrix_v) vs = PassShape{p.n_chunks, Hkv, p.chunk_tokens};
        else vs = PassShape{grouped ? p.n_chunks : group_grid_x(p.n_chunks, geo.G), grouped ? Hkv * (geo.G / group_heads(geo.G)) : Hkv,
                            p.chunk_tokens};
    }
    // task maps (per-sequence lengths): not for the swizzled grids of ungrouped multi-query heads
    const bool mapped = ragged && n_blocks > 0 && (geo.G == 1 || grouped || matrix) && task_map_fits(ks, B) && task_map_fits(vs, B);
    const bool v_mapped = mapped && (geo.G == 1 || grouped || matrix_v);
    StepGeom geo_k = geo, geo_v = geo;
    int *v_chunks = nullptr;
    if (mapped) geo_k.task_map = reinterpret_cast<const u32x2 *>(ws + lay.map_k);
    if (v_mapped) {
        geo_v.task_map = reinterpret_cast<const u32x2 *>(ws + lay.map_v);
        v_chunks = reinterpret_cast<int *>(ws + lay.v_chunks);
    }

    int persist = 1;
    bool k_prepared = false;     // the set-up of the matrix-core K pass was done by the first kernel
    if (ragged) {
        // per-sequence lengths live on the device: one small kernel appends every token and flushes the rest
        // buffers that fill up with it; its last 2*B workgroups write the task maps
        TaskMaps maps;
        maps.map_k = mapped ? reinterpret_cast<u32x2 *>(ws + lay.map_k) : nullptr;
        maps.map_v = v_mapped ? reinterpret_cast<u32x2 *>(ws + lay.map_v) : nullptr;
        maps.v_chunks = v_chunks;
        maps.k = ks;
        maps.v = vs;
        KPrepare prep = {q16, nullptr, k_levels_out, ref ? 1 : 0};
        if (n_blocks > 0 && matrix) prep.words = reinterpret_cast<u32 *>(ws + lay.prep);
        k_prepared = prep.words != nullptr;
        const int n_prep = k_prepared ? (B * Hkv + 3) / 4 : 0;
        hipLaunchKernelGGL((fused_pre_kernel<D>), dim3(B * Hkv * kPreSplit + n_prep + (mapped ? 2 * B : 0)), dim3(256), 0, st, kf8, km4,
                           kl4, vf8, vm4, vl4, k16, v16, rk16, rv16, kcm, vcm, geo, maps, B, prep);
        int rc = check_launch("decode_step(pre)");
        if (rc != AKV_OK) return rc;
        persist = 0;
    } else if (cur_len % cb + 1 == cb) {
        // the token fills the rest buffer: flush it into the planes before computing
        const int rest_start = cur_len / cb * cb;
        hipLaunchKernelGGL(fused_persist_kernel, dim3(B * Hkv), dim3(D < 256 ? D : 256), 0, st, k16, v16, rk16, rv16, kcm,
                           vcm, Hkv, D, cb, cur_len % cb);
        int rc = check_launch("decode_step(persist)");
        if (rc != AKV_OK) return rc;
        rc = launch_k_save_blocks(kf8, km4, kl4, restk, B, Hkv, 1, n_max_blocks, D, kb, rest_start, cb, st);
        if (rc != AKV_OK) return rc;
        rc = launch_v_save(vf8, vm4, vl4, restv, B, Hkv, max_seq_len, D, rest_start, cb, cb, st);
        if (rc != AKV_OK) return rc;
        persist = 0;
    }
    MiddleArgs ma;
    ma.q = q16; ma.k_new = k16; ma.v_new = v16;
    ma.mask = reinterpret_cast<const unsigned short *>(mask);
    ma.restk = rk16; ma.restv = rv16;
    ma.scores = s16; ma.probs = p16; ma.otail = otail;
    ma.kcm = kcm; ma.vcm = vcm; ma.toe = toe; ma.amin = amin; ma.v_first_8 = vf8;
    ma.g = geo; ma.mask_stride = mask_stride; ma.top_k = top_k; ma.persist = persist;
    ma.record_probs = (flags & AKV_STEP_NO_PROBS_RECORD) ? 0 : 1;
    mark(0, st);
    if (n_blocks > 0 && matrix) {
        int rc = AKV_OK;
        if constexpr (D <= 128)
            rc = launch_mfma_k_pass<D>(kf8, km4, kl4, kcm, q16, k16, s16, k_levels_out, reinterpret_cast<u32 *>(ws + lay.prep),
                                       geo_k, B, n_blocks, ref, scale, st, nullptr, k_prepared);
        if (rc != AKV_OK) return rc;
    } else if (n_blocks > 0 && grouped) {
        int rc = launch_group_k_pass<D>(kf8, km4, kl4, kcm, q16, k16, s16, k_levels_out, geo_k, B, n_blocks, ref, scale, st);
        if (rc != AKV_OK) return rc;
    } else if (n_blocks > 0 && kb == 256) {
        dim3 grid(ks.grid_x, ks.grid_y, B);
        if constexpr (D <= 128) {
#define AKV_KS(RF, UNI)                                                                                                      \
    hipLaunchKernelGGL((fused_k_pass256_split_kernel<D, RF, 4, UNI>), grid, dim3(256), 0, st, kf8, km4, kl4, kcm, q16, k16, s16, \
                       k_levels_out, geo_k, scale)
            const bool uniform = geo_k.seq_lens == nullptr && geo_k.task_map == nullptr;
            if (ref) { if (uniform) AKV_KS(true, true); else AKV_KS(true, false); }
            else { if (uniform) AKV_KS(false, true); else AKV_KS(false, false); }
#undef AKV_KS
        }
        int rc = check_launch("decode_step(k_pass256 split)");
        if (rc != AKV_OK) return rc;
    } else if (n_blocks > 0) {
        dim3 grid(ks.grid_x, ks.grid_y, B);
#define AKV_KP(RF, WH)                                                                                                 \
    hipLaunchKernelGGL((fused_k_pass_kernel<D, RF, WH>), grid, dim3(256), 0, st, kf8, km4, kl4, kcm, q16, k16, s16,   \
                       k_levels_out, geo_k, bpw, scale)
        bool launched = false;
        if constexpr (D <= 128) {
            if (k_whole) {
                if (geo_k.G == 1 && geo_k.seq_lens == nullptr && geo_k.task_map == nullptr) {
                    if (ref)
                        hipLaunchKernelGGL((fused_k_pass_kernel<D, true, true, true>), grid, dim3(256), 0, st, kf8, km4, kl4, kcm, q16,
                                           k16, s16, k_levels_out, geo_k, bpw, scale);
                    else
                        hipLaunchKernelGGL((fused_k_pass_kernel<D, false, true, true>), grid, dim3(256), 0, st, kf8, km4, kl4, kcm, q16,
                                           k16, s16, k_levels_out, geo_k, bpw, scale);
                } else {
                    if (ref) AKV_KP(true, true); else AKV_KP(false, true);
                }
                launched = true;
            }
        }
        if (!launched) {
            if (ref) AKV_KP(true, false); else AKV_KP(false, false);
        }
#undef AKV_KP
        int rc = check_launch("decode_step(k_pass)");
        if (rc != AKV_OK) return rc;
    }
    mark(1, st);
    // Second half of the step in one launch (see tail_step_kernel)
    // It is used when the (batch, head) pairs spread evenly over the compute units (every unit gets the same one or
    // two rows) and the rows are not long: measured on MI355X with 32 heads x 128, against the three launches it
    // replaces, us per step: 61.9 vs 72 at batch 8 x 4096 tokens, 76.4 vs 84.2 at 8 x 5120, 89.5 vs 96.9 at 8 x 6144,
    // 104.9 vs 110.6 at 8 x 7168, 125.9 vs 128.6 at 8 x 8192, 116.4 vs 127.7 at 16 x 4096, 143.9 vs 152.9 at 16 x 5120,
    // 169.8 vs 180.9 at 16 x 6144; with two rows of 8192 tokens per unit the V pass of many small workgroups was ahead
    // (241.5 vs 250.7 with an earlier form of the kernel), hence up to 12288 tokens per compute unit.
    // With fewer rows than compute units a row's workgroup streams alone at about 45 GB/s, while the V pass of many
    // small workgroups needs 4 us or the time of its bytes at 5 TB/s and then two more launches (2.5 us): measured
    // with 32 heads x 128 at batch 1 x 1024 tokens 15.9 vs 20.1 us per step, 2 x 2048: 21.0 vs 26.3, 4 x 4096: 39.2
    // vs 45.6, but 1 x 4096: 30.3 vs 23.8.
    const int cus = compute_units();
    const int rows = B * Hq;
    bool tail = cus > 0 && rows % cus == 0 && rows / cus <= tail_rows_per_cu && (rows / cus) * R <= 12288;
    if (cus > 0 && rows < cus) {
        const float row_us = (float)R * D / 45e3f, passes_us = fmaxf(4.f, (float)rows * R * D / 5e6f) + 2.5f;
        tail = row_us < passes_us;
    }
    // AKV_TUNE_TAIL=0/1 in the environment overrides the choice (the tests run both forms of the step on the same inputs)
    { AKV_TUNE("AKV_TUNE_TAIL", v); if (has_v) tail = v != 0; }
    tail = tail && n_blocks >= 1 && R <= tail_max_tokens && geo.G == 1 && !ragged && !(literal_broadcast && !ref);
    if (tail) {
        // (16 waves per workgroup measured 1 us slower than 8)
        if (ref) {
            hipLaunchKernelGGL((tail_step_ref_kernel<D, 4, 3, 512>), dim3(B * Hq), dim3(512), 0, st, vf8, vm4, vl4, ma,
                               reinterpret_cast<unsigned short *>(out), v_levels_out);
        } else {
            // Half tiles per wave that stream before the row's threshold is known (about what the probe's gather takes under
            // load), the first two of them requested between the phases of the softmax.  Measured at batch 8 x 32 heads x
            // 4096 tokens, second kernel alone by events: 27.4 us with 4 and none requested early, 25.7 with 4 and two
            // early, 25.5 with 5 and two, 25.8 with 5 and three.
            constexpr int fa = 5;
            if (ma.mask != nullptr)
                hipLaunchKernelGGL((tail_step_kernel<D, 512, 2, true>), dim3(B * Hq), dim3(512), 0, st, vf8, vm4, vl4, ma,
                                   reinterpret_cast<unsigned short *>(out), v_levels_out, amin_out, fa);
            else
                hipLaunchKernelGGL((tail_step_kernel<D, 512, 2, false>), dim3(B * Hq), dim3(512), 0, st, vf8, vm4, vl4, ma,
                                   reinterpret_cast<unsigned short *>(out), v_levels_out, amin_out, fa);
        }
        mark(2, st);
        mark(3, st);
        mark(4, st);
        mark(5, st);
        mark(6, st);
        return check_launch("decode_step(tail)");
    }
    {
        // threads per (batch, head) row: a thread keeps 32 scores in registers between the softmax passes, so
        // rows above 8192 / 16384 tokens get 512 / 1024 threads (512 and 1024 measure level with 256 at 4096 tokens for 256
        // rows; for 1024 rows of 2048 to 8192 tokens the stage takes 12.3 / 15.2 / 25.1 us with 256 / 512 / 1024)
        const int nt = R <= 8192 ? 256 : (R <= 16384 ? 512 : 1024);
        if (nt == 1024) hipLaunchKernelGGL((fused_middle_kernel<D, 1024>), dim3(B * Hq), dim3(1024), 0, st, ma);
        else if (nt == 512) hipLaunchKernelGGL((fused_middle_kernel<D, 512>), dim3(B * Hq), dim3(512), 0, st, ma);
        else hipLaunchKernelGGL((fused_middle_kernel<D, 256>), dim3(B * Hq), dim3(256), 0, st, ma);
    }
    int rc = check_launch("decode_step(middle)");
    if (rc != AKV_OK) return rc;
    if (literal_broadcast && !ref && R > 0) {
        hipLaunchKernelGGL(fused_amin_literal_kernel, dim3(B * Hq), dim3(64), 0, st, toe, vcm, amin, Hq, D);
        rc = check_launch("decode_step(amin)");
        if (rc != AKV_OK) return rc;
    }
    mark(2, st);
    if (p.n_chunks > 0 && matrix_v) {
        if constexpr (D <= 128)
            rc = launch_mfma_v_pass<D>(vf8, vm4, vl4, p16, amin, partial, v_levels_out, R, amin_out, geo_v, B, p, ref, st);
        if (rc != AKV_OK) return rc;
    } else if (p.n_chunks > 0 && grouped) {
        rc = launch_group_v_pass<D>(vf8, vm4, vl4, p16, amin, partial, v_levels_out, R, amin_out, geo_v, B, p, ref, st);
        if (rc != AKV_OK) return rc;
    } else if (p.n_chunks > 0) {
        dim3 grid(group_grid_x(p.n_chunks, geo.G), Hkv, B);
        const bool uniform_v = geo_v.G == 1 && geo_v.seq_lens == nullptr && geo_v.task_map == nullptr;
#define AKV_VP1(RF, N, UNI)                                                                                               \
    hipLaunchKernelGGL((fused_v_pass_kernel<D, RF, N, UNI>), grid, dim3(256), 0, st, vf8, vm4, vl4, p16, amin, partial,   \
                       v_levels_out, R, amin_out, geo_v, p.tokens_per_wave, p.n_chunks)
#define AKV_VP(RF, N)                                                                                                     \
    do {                                                                                                                  \
        if (uniform_v) AKV_VP1(RF, N, true);                                                                              \
        else AKV_VP1(RF, N, false);                                                                                       \
    } while (0)
        if (ref) {
            if (p.iters_per_wave == 1) AKV_VP(true, 1);
            else if (p.iters_per_wave == 2) AKV_VP(true, 2);
            else AKV_VP(true, 4);
        } else {
            if (p.iters_per_wave == 1) AKV_VP(false, 1);
            else if (p.iters_per_wave == 2) AKV_VP(false, 2);
            else AKV_VP(false, 4);
        }
#undef AKV_VP
#undef AKV_VP1
        rc = check_launch("decode_step(v_pass)");
        if (rc != AKV_OK) return rc;
    }
    mark(3, st);
    hipLaunchKernelGGL(fused_combine_kernel, dim3(B * Hq), dim3(D < 256 ? D : 256), 0, st, partial, otail,
                       reinterpret_cast<unsigned short *>(out), D, p.n_chunks, seq_lens, Hq, v_chunks);
    mark(4, st);
    mark(5, st);
    mark(6, st);
    return check_launch("decode_step(combine)");
}

}  // namespace akv

using namespace akv;

extern "C" int akv_profile_enable(int enable) {
    if (enable && !g_ev_ready) {
        for (int i = 0; i < 7; ++i) {
            if (hipEventCreate(&g_ev[i]) != hipSuccess) {
                set_error("profile_enable: hipEventCreate failed");
                return AKV_ERR_LAUNCH;
            }
        }
        g_ev_ready = true;
    }
    g_profile = enable != 0;
    return AKV_OK;
}

extern "C" int akv_profile_read(float *phase_ms) {
    AKV_REQUIRE(phase_ms != nullptr && g_ev_ready, "profile_read: profiling was never enabled");
    if (hipEventSynchronize(g_ev[4]) != hipSuccess) {
        set_error("profile_read: no completed step to read");
        return AKV_ERR_LAUNCH;
    }
    for (int i = 0; i < 4; ++i) {
        if (hipEventElapsedTime(&phase_ms[i], g_ev[i], g_ev[i + 1]) != hipSuccess) {
            set_error("profile_read: hipEventElapsedTime failed");
            return AKV_ERR_LAUNCH;
        }
    }
    return AKV_OK;
}

extern "C" int akv_profile_read_empty(float *empty_ms) {
    AKV_REQUIRE(empty_ms != nullptr && g_ev_ready, "profile_read_empty: profiling was never enabled");
    if (hipEventSynchronize(g_ev[6]) != hipSuccess || hipEventElapsedTime(empty_ms, g_ev[5], g_ev[6]) != hipSuccess) {
        set_error("profile_read_empty: no completed step to read");
        return AKV_ERR_LAUNCH;
    }
    return AKV_OK;
}

extern "C" size_t akv_decode_step_workspace_bytes(int bsz, int n_q_heads, int head_dim, int max_seq_len) {
    if (bsz <= 0 || n_q_heads <= 0 || head_dim <= 0 || max_seq_len <= 0) return 0;
    return step_layout(bsz, n_q_heads, head_dim, max_seq_len).total;
}

extern "C" int akv_decode_step_gqa(uint8_t *k_first_8, uint8_t *k_mid_4, uint8_t *k_last_4, uint8_t *v_first_8,
                                   uint8_t *v_mid_4, uint8_t *v_last_4, uint8_t *k_exp_column_max,
                                   uint8_t *v_exp_column_max, uint8_t *restk, uint8_t *restv, const uint8_t *q,
                                   const uint8_t *k_new, const uint8_t *v_new, const uint8_t *mask, int mask_stride,
                                   uint8_t *out, uint8_t *scores, uint8_t *probs, int row_stride, void *workspace,
                                   size_t workspace_bytes, uint8_t *k_levels_out, uint8_t *v_levels_out,
                                   uint8_t *amin_out, int bsz, int n_q_heads, int n_kv_heads, int n_max_blocks,
                                   int max_seq_len, int head_dim, int d_block, int k_block, int top_max_k, int cur_len,
                                   int *seq_lens, int reference, int literal_broadcast, akv_stream_t stream) {
    AKV_REQUIRE(k_first_8 && k_mid_4 && k_last_4 && v_first_8 && v_mid_4 && v_last_4 && k_exp_column_max &&
                    v_exp_column_max && restk && restv && q && k_new && v_new && out && scores && probs && workspace,
                "decode_step: null pointer");
    AKV_REQUIRE(bsz > 0 && n_q_heads > 0 && n_kv_heads > 0 && n_max_blocks > 0 && max_seq_len > 0,
                "decode_step: non-positive dimension");
    AKV_REQUIRE(n_q_heads % n_kv_heads == 0, "decode_step: %d query heads are not a multiple of %d KV heads", n_q_heads,
                n_kv_heads);
    AKV_REQUIRE(head_dim == 64 || head_dim == 128 || head_dim == 256,
                "decode_step: head_dim %d not supported by the fused step (64, 128, 256); use the five ops", head_dim);
    AKV_REQUIRE(d_block == 64, "decode_step: d_block %d not supported by the fused step (64); use the five ops", d_block);
    AKV_REQUIRE(k_block == 64 || (k_block == 256 && head_dim <= 128 && n_q_heads / n_kv_heads <= 16),
                "decode_step: k_block %d: K plane blocks are 64 tokens, or 256 for head_dim 64 or 128 and at most 16 query "
                "heads per KV head", k_block);
    AKV_REQUIRE(top_max_k == 32, "decode_step: top_max_k %d not supported by the fused step (32)", top_max_k);
    AKV_REQUIRE(bsz <= 65535 && n_kv_heads <= 65535, "decode_step: bsz/heads exceed the grid limit 65535");
    AKV_REQUIRE(cur_len >= 0 && cur_len + 1 <= max_seq_len, "decode_step: cache full (%d of %d tokens)", cur_len, max_seq_len);
    AKV_REQUIRE((literal_broadcast & ~(AKV_STEP_LITERAL_BROADCAST | AKV_STEP_NO_PROBS_RECORD)) == 0, "decode_step: unknown flags %d", literal_broadcast);
    AKV_REQUIRE(!(literal_broadcast & AKV_STEP_LITERAL_BROADCAST) || (n_q_heads == n_kv_heads && seq_lens == nullptr),
                "decode_step: literal_broadcast is defined for multi-head caches of uniform length only");
    const int flushed = (cur_len + 1) / d_block * d_block;
    AKV_REQUIRE(flushed + d_block <= 65536 * 32, "decode_step: at most %d flushed tokens (16-bit group index of the probe)",
                65536 * 32);
    AKV_REQUIRE((int64_t)n_max_blocks * k_block >= flushed, "decode_step: K planes hold %d blocks of %d, %d tokens flushed",
                n_max_blocks, k_block, flushed);
    AKV_REQUIRE(row_stride % 8 == 0 && row_stride >= flushed + d_block,
                "decode_step: row_stride %d must be a multiple of 8 and >= %d", row_stride, flushed + d_block);
    AKV_REQUIRE(mask == nullptr || mask_stride == 0 || mask_stride >= cur_len + 1,
                "decode_step: mask row stride %d shorter than %d (0 = one row for all sequences)", mask_stride, cur_len + 1);
    AKV_REQUIRE((int64_t)max_seq_len * head_dim < (int64_t)1 << 31 && (int64_t)n_max_blocks * head_dim * k_block < (int64_t)1 << 31,
                "decode_step: one (batch, head) slice of a high-byte plane must stay below 2 GiB");
    const size_t need = akv_decode_step_workspace_bytes(bsz, n_q_heads, head_dim, max_seq_len);
    AKV_REQUIRE(workspace_bytes >= need, "decode_step: workspace of %zu bytes, %zu needed", workspace_bytes, need);
    AKV_REQUIRE(((uintptr_t)workspace & 255) == 0 && ((uintptr_t)scores & 15) == 0 && ((uintptr_t)probs & 15) == 0,
                "decode_step: workspace must be 256-byte aligned, scores/probs 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    uint8_t *ws = static_cast<uint8_t *>(workspace);
#define AKV_STEP(DD)                                                                                                  \
    return run_step<DD>(k_first_8, k_mid_4, k_last_4, v_first_8, v_mid_4, v_last_4, k_exp_column_max, v_exp_column_max, \
                        restk, restv, q, k_new, v_new, mask, mask_stride, out, scores, probs, row_stride, ws,          \
                        k_levels_out, v_levels_out, amin_out, bsz, n_q_heads, n_kv_heads, n_max_blocks, max_seq_len,   \
                        d_block, k_block, top_max_k, cur_len, seq_lens, reference != 0, literal_broadcast, st);
    if (head_dim == 64) { AKV_STEP(64) }
    if (head_dim == 128) { AKV_STEP(128) }
    AKV_STEP(256)
#undef AKV_STEP
}

extern "C" int akv_decode_step_desc(const akv_step_desc *d, const uint8_t *q, const uint8_t *k_new, const uint8_t *v_new,
                                    const uint8_t *mask, int mask_stride, uint8_t *out, uint8_t *k_levels_out,
                                    uint8_t *v_levels_out, uint8_t *amin_out, int cur_len, int *seq_lens, int reference,
                                    int literal_broadcast, akv_stream_t stream) {
    AKV_REQUIRE(d != nullptr, "decode_step: null descriptor");
    return akv_decode_step_gqa(d->k_first_8, d->k_mid_4, d->k_last_4, d->v_first_8, d->v_mid_4, d->v_last_4, d->k_exp_column_max,
                               d->v_exp_column_max, d->restk, d->restv, q, k_new, v_new, mask, mask_stride, out, d->scores,
                               d->probs, d->row_stride, d->workspace, d->workspace_bytes, k_levels_out, v_levels_out, amin_out,
                               d->bsz, d->n_q_heads, d->n_kv_heads, d->n_max_blocks, d->max_seq_len, d->head_dim, d->d_block,
                               d->k_block, d->top_max_k, cur_len, seq_lens, reference, literal_broadcast, stream);
}

extern "C" int akv_decode_step(uint8_t *k_first_8, uint8_t *k_mid_4, uint8_t *k_last_4, uint8_t *v_first_8,
                               uint8_t *v_mid_4, uint8_t *v_last_4, uint8_t *k_exp_column_max,
                               uint8_t *v_exp_column_max, uint8_t *restk, uint8_t *restv, const uint8_t *q,
                               const uint8_t *k_new, const uint8_t *v_new, const uint8_t *mask, int mask_stride,
                               uint8_t *out, uint8_t *scores, uint8_t *probs, int row_stride, void *workspace,
                               size_t workspace_bytes, uint8_t *k_levels_out, uint8_t *v_levels_out, uint8_t *amin_out,
                               int bsz, int n_kv_heads, int n_max_blocks, int max_seq_len, int head_dim, int d_block,
                               int top_max_k, int cur_len, int rest_start, int rest_len, int reference,
                               int literal_broadcast, akv_stream_t stream) {
    AKV_REQUIRE(d_block > 0 && cur_len >= 0 && rest_start >= 0 && rest_len >= 0 && rest_len < d_block &&
                    rest_start % d_block == 0 && rest_start + rest_len == cur_len,
                "decode_step: inconsistent state cur_len=%d rest_start=%d rest_len=%d", cur_len, rest_start, rest_len);
    return akv_decode_step_gqa(k_first_8, k_mid_4, k_last_4, v_first_8, v_mid_4, v_last_4, k_exp_column_max,
                               v_exp_column_max, restk, restv, q, k_new, v_new, mask, mask_stride, out, scores, probs,
                               row_stride, workspace, workspace_bytes, k_levels_out, v_levels_out, amin_out, bsz,
                               n_kv_heads, n_kv_heads, n_max_blocks, max_seq_len, head_dim, d_block, d_block, top_max_k,
                               cur_len, nullptr, reference, literal_broadcast, stream);
}

// ------------------------------------------------------------------------------------------------
// The step for callers that cannot allocate: its workspace (probe exponents, thresholds, tail outputs, partial sums
// of the V pass, set-up words and task maps) lives in a file-scope device array instead of a buffer the caller
// brings.  Every GPU the library runs on holds its own copy of the array at its own address; the address is looked
// up once per device and only that pointer is ever handed to kernels.
// ------------------------------------------------------------------------------------------------
constexpr size_t kStaticScratchBytes = AKV_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices];   // per device: address of that device's copy of `scratch`

// address of the current device's copy of the scratch array (null + error set on failure)
void *static_scratch() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error("decode_step_static: no current device (or more than %d devices)", kMaxDevices);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr) {
            set_error("decode_step_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = p;
    }
    return g_scratch_ptr[dev];
}
}  // namespace

extern "C" int akv_decode_step_static(uint8_t *k_first_8, uint8_t *k_mid_4, uint8_t *k_last_4, uint8_t *v_first_8,
                                      uint8_t *v_mid_4, uint8_t *v_last_4, uint8_t *k_exp_column_max,
                                      uint8_t *v_exp_column_max, uint8_t *restk, uint8_t *restv, const uint8_t *q,
                                      const uint8_t *k_new, const uint8_t *v_new, const uint8_t *mask, int mask_stride,
                                      uint8_t *out, uint8_t *scores, uint8_t *probs, int row_stride,
                                      uint8_t *k_levels_out, uint8_t *v_levels_out, uint8_t *amin_out, int bsz,
                                      int n_kv_heads, int n_max_blocks, int max_seq_len, int head_dim, int d_block,
                                      int top_max_k, int cur_len, int rest_start, int rest_len, int reference,
                                      int literal_broadcast, akv_stream_t stream) {
    const size_t need = akv_decode_step_workspace_bytes(bsz, n_kv_heads, head_dim, max_seq_len);
    AKV_REQUIRE(need > 0, "decode_step_static: non-positive dimension");
    AKV_REQUIRE(need <= kStaticScratchBytes,
                "decode_step_static: this shape needs %zu bytes of workspace, the built-in scratch array holds %zu; use "
                "akv_decode_step with a workspace of your own", need, kStaticScratchBytes);
    void *ws = static_scratch();
    if (ws == nullptr) return AKV_ERR_LAUNCH;
    return akv_decode_step(k_first_8, k_mid_4, k_last_4, v_first_8, v_mid_4, v_last_4, k_exp_column_max, v_exp_column_max,
                           restk, restv, q, k_new, v_new, mask, mask_stride, out, scores, probs, row_stride, ws,
                           kStaticScratchBytes, k_levels_out, v_levels_out, amin_out, bsz, n_kv_heads, n_max_blocks,
                           max_seq_len, head_dim, d_block, top_max_k, cur_len, rest_start, rest_len, reference,
                           literal_broadcast, stream);
}

