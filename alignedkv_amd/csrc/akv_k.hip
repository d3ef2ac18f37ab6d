// K side of the AlignedKV hot path: plane writes (k_cache_save) and decode scores (k_cache_compute).
//
// Plane layout (reference: extension/k_cache_file.py:45-53): per (batch, head, block) a block of
// d_block tokens is stored channel-major, first_8[d][slot] (d_block bytes per channel) and
// mid_4/last_4[d][slot/2] (d_block/2 bytes per channel, even slot in the high nibble).
//
// Score kernel, tuned shape (d_block == 64, d_head in {64,128,256}): one wave owns one block.
// A 16-byte load per lane covers 16 channels x 64 slots of first_8 (lane = 16 slots of one
// channel), an 8-byte load per lane covers the same (channel, slots) of a nibble plane, so the
// three planes of an element meet in one lane without any exchange.  The fetch level depends
// only on the channel, i.e. on (load group, lane/4): nibble loads of skipped channels are issued
// with an out-of-range buffer offset (they return 0 and fetch nothing) and OR-ed with the
// substitution byte.  Each lane keeps 16 fp32 accumulators (its 16 slots); a reduce-scatter over
// the 16 lanes that share the slots leaves one score per lane.
#include "akv_cores.h"

namespace akv {

// ------------------------------------------------------------------------------------------------
// k_cache_save
// ------------------------------------------------------------------------------------------------
// grid (n_blocks * tiles_per_block, H, B), 256 threads; a workgroup transposes one tile of up to
// 64 slots through LDS (dynamic LDS = tile_slots * (D + 2) halves) so that both the token-major
// fp16 reads and the channel-major plane writes are coalesced.
// reference: extension/csrc/K_cache.cu:19-58 (same destination bytes, written instead of accumulated).
__global__ __launch_bounds__(256) void k_save_blocks_kernel(
    uint8_t *__restrict__ first_8, uint8_t *__restrict__ mid_4, uint8_t *__restrict__ last_4,
    const unsigned short *__restrict__ k_new, int n_max_blocks, int H, int D, int cb, int tile_slots,
    int start_pos, int n_tokens, int seqlen, int first_tile) {
    extern __shared__ unsigned short tile[];   // [tile_slots][D + 2]
    const int pitch = D + 2;
    const int h = blockIdx.y, b = blockIdx.z;
    const int t0 = (first_tile + blockIdx.x) * tile_slots;        // first source token of this tile
    const int pos = start_pos + t0;                               // its position in the cache (a multiple of tile_slots)
    const int z = pos / cb, slot0 = pos - z * cb;                 // destination block and first slot in it
    const int nv = min(tile_slots, n_tokens - t0);                // valid tokens of this tile
    if (nv <= 0) return;
    const int halfD = D >> 1;
    const u32 *src32 = reinterpret_cast<const u32 *>(k_new);
    for (int idx = threadIdx.x; idx < nv * halfD; idx += blockDim.x) {
        int j = idx / halfD, dp = idx - j * halfD;
        u32 w = src32[(((int64_t)b * seqlen + t0 + j) * H + h) * halfD + dp];
        tile[j * pitch + 2 * dp] = (unsigned short)(w & 0xffffu);
        tile[j * pitch + 2 * dp + 1] = (unsigned short)(w >> 16);
    }
    __syncthreads();
    const int64_t blk_base = (((int64_t)b * H + h) * n_max_blocks + z) * (int64_t)D * (cb >> 1);
    uint8_t *f8 = first_8 + blk_base * 2 + slot0;
    uint8_t *m4 = mid_4 + blk_base + (slot0 >> 1);
    uint8_t *l4 = last_4 + blk_base + (slot0 >> 1);
    // first_8: 4 slots per thread
    const int q4 = tile_slots >> 2;
    for (int idx = threadIdx.x; idx < D * q4; idx += blockDim.x) {
        int d = idx / q4, j = (idx - d * q4) * 4;
        if (j + 3 < nv) {
            u32 w = (u32)(tile[j * pitch + d] >> 8) | ((u32)(tile[(j + 1) * pitch + d] >> 8) << 8) |
                    ((u32)(tile[(j + 2) * pitch + d] >> 8) << 16) | ((u32)(tile[(j + 3) * pitch + d] >> 8) << 24);
            *reinterpret_cast<u32 *>(f8 + (int64_t)d * cb + j) = w;
        } else {
            for (int jj = j; jj < nv; ++jj) f8[(int64_t)d * cb + jj] = (uint8_t)(tile[jj * pitch + d] >> 8);
        }
    }
    // nibble planes: 8 slots (4 bytes) per thread
    const int q8 = tile_slots >> 3;
    for (int idx = threadIdx.x; idx < D * q8; idx += blockDim.x) {
        int d = idx / q8, j = (idx - d * q8) * 8;
        if (j >= nv) continue;
        u32 mw = 0, lw = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int je = j + 2 * i, jo = je + 1;
            u32 le = je < nv ? (tile[je * pitch + d] & 0xffu) : 0u;
            u32 lo = jo < nv ? (tile[jo * pitch + d] & 0xffu) : 0u;
            mw |= ((le & 0xf0u) | (lo >> 4)) << (8 * i);
            lw |= (((le & 0x0fu) << 4) | (lo & 0x0fu)) << (8 * i);
        }
        if (j + 7 < nv) {
            *reinterpret_cast<u32 *>(m4 + (int64_t)d * (cb >> 1) + (j >> 1)) = mw;
            *reinterpret_cast<u32 *>(l4 + (int64_t)d * (cb >> 1) + (j >> 1)) = lw;
        } else {
            int nbytes = (nv - j + 1) >> 1;
            for (int i = 0; i < nbytes; ++i) {
                m4[(int64_t)d * (cb >> 1) + (j >> 1) + i] = (uint8_t)(mw >> (8 * i));
                l4[(int64_t)d * (cb >> 1) + (j >> 1) + i] = (uint8_t)(lw >> (8 * i));
            }
        }
    }
}

// The same bytes for whole tiles of ts tokens (64, 128 or 256: as many as divide the block) when D is a multiple of 8 and
// everything is 16-byte aligned.  LDS holds the tile as it comes (16-byte vectors of 8 channels of one token) and is
// read back in the same vectors, 8 tokens x 8 channels per thread, which the thread turns into the plane words of its 8
// channels in registers: 16 LDS operations of 16 bytes per 128 elements instead of 96 of 2 bytes.  The vector index
// within a token's row is XOR-ed with a function of the token so that the reads spread over the banks.  Thread
// (o, jg) = (channel octet, group of 8 slots): the ts/8 threads of an octet write ts contiguous bytes of each first_8
// row and ts/2 of each nibble row -- with blocks of 256 tokens a whole row at once (tiles of 64 slots left every 128-byte
// line to four workgroups: 2.8 TB/s read + write, against 4.3 with blocks of 64 tokens).
// A workgroup takes dc of the D channels.  grid (tiles * D / dc, H, B); ts * dc / 64 threads; dynamic LDS 2 ts dc bytes.
__global__ __launch_bounds__(256) void k_save_tiles_kernel(uint8_t *__restrict__ first_8, uint8_t *__restrict__ mid_4,
                                                          uint8_t *__restrict__ last_4, const u32x4 *__restrict__ k_new,
                                                          int n_max_blocks, int H, int D, int cb, int ts, int dc, int start_pos,
                                                          int first_token, int seqlen) {
    extern __shared__ u32x4 tile_vec[];        // [ts tokens][dc / 8 vectors]
    const int octs = D >> 3, wo = dc >> 3;     // vectors per token: in memory, in this workgroup's share
    const int chunks = D / dc;
    const int tile_idx = blockIdx.x / chunks, chunk = blockIdx.x - tile_idx * chunks;
    const int swz = (wo & (wo - 1)) == 0 ? wo - 1 : 0;
    const int swz_mul = wo >= 16 ? 2 : 1;
    const int h = blockIdx.y, b = blockIdx.z;
    const int t0 = first_token + tile_idx * ts;
    const int pos = start_pos + t0;
    const int z = pos / cb, slot0 = pos - z * cb;
    for (int idx = threadIdx.x; idx < ts * wo; idx += blockDim.x) {
        const int j = idx / wo, o = idx - j * wo;
        tile_vec[j * wo + (o ^ (((j >> 3) * swz_mul) & swz))] = k_new[(((int64_t)b * seqlen + t0 + j) * H + h) * octs + chunk * wo + o];
    }
    __syncthreads();
    const int64_t blk_base = (((int64_t)b * H + h) * n_max_blocks + z) * (int64_t)D * (cb >> 1);
    uint8_t *f8 = first_8 + blk_base * 2 + slot0;
    uint8_t *m4 = mid_4 + blk_base + (slot0 >> 1);
    uint8_t *l4 = last_4 + blk_base + (slot0 >> 1);
    const int groups = ts >> 3;
    for (int task = threadIdx.x; task < groups * wo; task += blockDim.x) {
        const int o = task / groups, jg = task - o * groups;
        u32 x[8][4];                           // [token 8 jg + i][channel pair c]: channels 8 o + 2 c (low half), + 1 (high half)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const u32x4 v = tile_vec[(8 * jg + i) * wo + (o ^ ((jg * swz_mul) & swz))];
            x[i][0] = v.x; x[i][1] = v.y; x[i][2] = v.z; x[i][3] = v.w;
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            // high bytes: [even channel of token a, of token b, odd channel of token a, of token b]
            const u32 h01 = __builtin_amdgcn_perm(x[1][c], x[0][c], 0x07030501u), h23 = __builtin_amdgcn_perm(x[3][c], x[2][c], 0x07030501u);
            const u32 h45 = __builtin_amdgcn_perm(x[5][c], x[4][c], 0x07030501u), h67 = __builtin_amdgcn_perm(x[7][c], x[6][c], 0x07030501u);
            // low bytes of the even slots and of the odd slots, same arrangement
            const u32 e02 = __builtin_amdgcn_perm(x[2][c], x[0][c], 0x06020400u), e46 = __builtin_amdgcn_perm(x[6][c], x[4][c], 0x06020400u);
            const u32 o13 = __builtin_amdgcn_perm(x[3][c], x[1][c], 0x06020400u), o57 = __builtin_amdgcn_perm(x[7][c], x[5][c], 0x06020400u);
#pragma unroll
            for (int par = 0; par < 2; ++par) {
                const u32 sel = par ? 0x07060302u : 0x05040100u;
                const int ch = chunk * dc + 8 * o + 2 * c + par;
                u32x2 hw;
                hw.x = __builtin_amdgcn_perm(h23, h01, sel);       // slots 8 jg + 0..3
                hw.y = __builtin_amdgcn_perm(h67, h45, sel);       // slots 8 jg + 4..7
                const u32 ev = __builtin_amdgcn_perm(e46, e02, sel);   // low bytes of slots 0, 2, 4, 6
                const u32 od = __builtin_amdgcn_perm(o57, o13, sel);   // of slots 1, 3, 5, 7
                const u32 mw = (ev & 0xF0F0F0F0u) | ((od >> 4) & 0x0F0F0F0Fu);
                const u32 lw = ((ev << 4) & 0xF0F0F0F0u) | (od & 0x0F0F0F0Fu);
                *reinterpret_cast<u32x2 *>(f8 + (int64_t)ch * cb + 8 * jg) = hw;
                *reinterpret_cast<u32 *>(m4 + (int64_t)ch * (cb >> 1) + 4 * jg) = mw;
                *reinterpret_cast<u32 *>(l4 + (int64_t)ch * (cb >> 1) + 4 * jg) = lw;
            }
        }
    }
}

// One token into slot `slot` of block `blk`: nibble insert (the other nibble of the byte is kept).
// grid (H, B), D threads.  reference: extension/csrc/K_cache.cu:63-94.
__global__ void k_save_token_kernel(uint8_t *__restrict__ first_8, uint8_t *__restrict__ mid_4,
                                    uint8_t *__restrict__ last_4, const unsigned short *__restrict__ k_new,
                                    int n_max_blocks, int H, int D, int cb, int blk, int slot) {
    const int h = blockIdx.x, b = blockIdx.y;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        u32 bits = k_new[((int64_t)b * H + h) * D + d];
        int64_t base = ((((int64_t)b * H + h) * n_max_blocks + blk) * D + d) * (int64_t)(cb >> 1);
        first_8[base * 2 + slot] = (uint8_t)(bits >> 8);
        uint8_t *pm = mid_4 + base + (slot >> 1);
        uint8_t *pl = last_4 + base + (slot >> 1);
        u32 mid = (bits >> 4) & 0xfu, last = bits & 0xfu;
        if (slot & 1) {
            *pm = (uint8_t)((*pm & 0xf0u) | mid);
            *pl = (uint8_t)((*pl & 0xf0u) | last);
        } else {
            *pm = (uint8_t)((*pm & 0x0fu) | (mid << 4));
            *pl = (uint8_t)((*pl & 0x0fu) | (last << 4));
        }
    }
}

// ------------------------------------------------------------------------------------------------
// k_cache_compute, tuned: d_block == 64
// grid (ceil(n_blocks / (4*blocks_per_wave)), H, B), 256 threads (4 waves).
// ------------------------------------------------------------------------------------------------
// WHOLE (head_dim 64 and 128, blocks_per_wave == 1): a wave requests all rows of its block at once instead of walking
// it in double-buffered half tiles (k_score_block_whole).
template <int D, bool REF, bool WHOLE = false>
__global__ __launch_bounds__(256) void k_compute_cb64_kernel(
    const uint8_t *__restrict__ first_8, const uint8_t *__restrict__ mid_4, const uint8_t *__restrict__ last_4,
    const uint8_t *__restrict__ sum_u8, const uint8_t *__restrict__ max_u8, const unsigned short *__restrict__ q,
    unsigned short *__restrict__ s, uint8_t *__restrict__ levels_out, int n_blocks, int n_max_blocks, int H,
    int blocks_per_wave, float scale) {
    constexpr int CB = 64;
    constexpr int NG = D / 16;
    const int lane = threadIdx.x & 63, wave = wave_index();
    const int h = blockIdx.y, b = blockIdx.z;
    const int bh = b * H + h;
    const int first_blk = (blockIdx.x * 4 + wave) * blocks_per_wave;
    if (first_blk >= n_blocks) return;
    const int end_blk = min(first_blk + blocks_per_wave, n_blocks);

    const int64_t plane_off = (int64_t)bh * n_max_blocks * (D * (CB / 2));
    KHalfTile<WHOLE ? D / 16 : D / 32> ta;
    if constexpr (WHOLE) {
        k_issue_half_h<D, D / 16>(ta, make_rsrc(first_8 + plane_off * 2, (u32)n_blocks * (D * CB)), first_blk, 0);
        __builtin_amdgcn_sched_barrier(0);
    } else {
        k_prefetch_first<D>(ta, first_8 + plane_off * 2, n_blocks, first_blk);
    }
    // per-lane channel data: channel of group g is g*16 + lane/4
    float qf[NG];
    u32 need_mid = 0, need_last = 0;
    const unsigned char mx = REF ? 0 : max_u8[bh];
#pragma unroll
    for (int g = 0; g < NG; ++g) {
        int c = g * 16 + (lane >> 2);
        qf[g] = half_bits_to_float(q[(int64_t)bh * D + c]);
        int lv = REF ? 0 : k_level(mx, sum_u8[(int64_t)bh * D + c]);
        need_mid |= (lv < 2 ? 1u : 0u) << g;
        need_last |= (lv == 0 ? 1u : 0u) << g;
        if (levels_out != nullptr && blockIdx.x == 0 && wave == 0 && (lane & 3) == 0)
            levels_out[(int64_t)bh * D + c] = (uint8_t)lv;
    }
    if constexpr (WHOLE) {
        k_score_block_whole<D>(ta, mid_4 + plane_off, last_4 + plane_off, n_blocks, first_blk, qf, need_mid, need_last,
                               s + (int64_t)bh * ((int64_t)(n_blocks + 1) * CB), scale);
    } else {
        k_score_blocks<D>(ta, first_8 + plane_off * 2, mid_4 + plane_off, last_4 + plane_off, n_blocks, first_blk, end_blk, qf,
                          need_mid, need_last, s + (int64_t)bh * ((int64_t)(n_blocks + 1) * CB), scale);
    }
}

// ------------------------------------------------------------------------------------------------
// k_cache_compute, tuned: d_block == 256 (see k256_score_blocks).
// grid (ceil(n_blocks / (4*blocks_per_wave)), H, B), 256 threads (4 waves).
// ------------------------------------------------------------------------------------------------
template <int D, bool REF>
__global__ __launch_bounds__(256) void k_compute_cb256_kernel(
    const uint8_t *__restrict__ first_8, const uint8_t *__restrict__ mid_4, const uint8_t *__restrict__ last_4,
    const uint8_t *__restrict__ sum_u8, const uint8_t *__restrict__ max_u8, const unsigned short *__restrict__ q,
    unsigned short *__restrict__ s, uint8_t *__restrict__ levels_out, int n_blocks, int n_max_blocks, int H,
    int blocks_per_wave, float scale) {
    constexpr int CB = 256;
    constexpr int NG = D / 4;
    const int lane = threadIdx.x & 63, wave = wave_index();
    const int h = blockIdx.y, b = blockIdx.z;
    const int bh = b * H + h;
    const int first_blk = (blockIdx.x * 4 + wave) * blocks_per_wave;
    if (first_blk >= n_blocks) return;
    const int end_blk = min(first_blk + blocks_per_wave, n_blocks);
    const int64_t plane_off = (int64_t)bh * n_max_blocks * (D * (CB / 2));
    KHalfTile<4> ta;
    k256_prefetch_first<D>(ta, first_8 + plane_off * 2, n_blocks, first_blk);
    // per-lane channel data: channel of group g is 4 g + lane/16
    u32 qh[NG / 2];
    u32 need_mid = 0, need_last = 0;
    const unsigned char mx = REF ? 0 : max_u8[bh];
#pragma unroll
    for (int g = 0; g < NG; ++g) {
        const int c = 4 * g + (lane >> 4);
        const u32 qb = q[(int64_t)bh * D + c];
        if (g & 1) qh[g >> 1] |= qb << 16; else qh[g >> 1] = qb;
        const int lv = REF ? 0 : k_level(mx, sum_u8[(int64_t)bh * D + c]);
        need_mid |= (lv < 2 ? 1u : 0u) << g;
        need_last |= (lv == 0 ? 1u : 0u) << g;
        if (levels_out != nullptr && blockIdx.x == 0 && wave == 0 && (lane & 15) == 0)
            levels_out[(int64_t)bh * D + c] = (uint8_t)lv;
    }
    k256_score_blocks<D>(ta, first_8 + plane_off * 2, mid_4 + plane_off, last_4 + plane_off, n_blocks, first_blk, end_blk, qh,
                         need_mid, need_last, s + (int64_t)bh * ((int64_t)(n_blocks + 1) * CB), n_blocks * CB, scale);
}

// ------------------------------------------------------------------------------------------------
// k_cache_compute, any shape: one thread per slot pair, like the reference's launch
// (extension/csrc/K_cache.cu:350-351) but with fp32 accumulation.
// grid (n_blocks, H, B), d_block/2 threads.
// ------------------------------------------------------------------------------------------------
template <bool REF>
__global__ void k_compute_generic_kernel(const uint8_t *__restrict__ first_8, const uint8_t *__restrict__ mid_4,
                                         const uint8_t *__restrict__ last_4, const uint8_t *__restrict__ sum_u8,
                                         const uint8_t *__restrict__ max_u8, const unsigned short *__restrict__ q,
                                         unsigned short *__restrict__ s, uint8_t *__restrict__ levels_out,
                                         int n_blocks, int n_max_blocks, int H, int D, int cb, float scale) {
    const int z = blockIdx.x, h = blockIdx.y, b = blockIdx.z, tx = threadIdx.x;
    const int bh = b * H + h;
    const unsigned char mx = REF ? 0 : max_u8[bh];
    const int64_t base = ((int64_t)bh * n_max_blocks + z) * (int64_t)D * (cb >> 1);
    float r1 = 0.f, r2 = 0.f;
    for (int i = 0; i < D; ++i) {
        int lv = REF ? 0 : k_level(mx, sum_u8[(int64_t)bh * D + i]);
        if (levels_out != nullptr && z == 0 && tx == 0) levels_out[(int64_t)bh * D + i] = (uint8_t)lv;
        int64_t row = base + (int64_t)i * (cb >> 1);
        u32 h1 = first_8[row * 2 + 2 * tx], h2 = first_8[row * 2 + 2 * tx + 1];
        u32 m = lv < 2 ? mid_4[row + tx] : 0u;
        u32 l = lv == 0 ? last_4[row + tx] : 0u;
        float qf = half_bits_to_float(q[(int64_t)bh * D + i]);
        r1 = fmaf(half_bits_to_float(rebuild_bits(h1, m >> 4, l >> 4, lv)), qf, r1);
        r2 = fmaf(half_bits_to_float(rebuild_bits(h2, m & 0xfu, l & 0xfu, lv)), qf, r2);
    }
    unsigned short *s_row = s + (int64_t)bh * ((int64_t)(n_blocks + 1) * cb);
    s_row[z * cb + 2 * tx] = float_to_half_bits(r1 * scale);
    s_row[z * cb + 2 * tx + 1] = float_to_half_bits(r2 * scale);
}

template <int D, bool REF>
static void launch_k_cb64(const uint8_t *f8, const uint8_t *m4, const uint8_t *l4, const uint8_t *sum_u8,
                          const uint8_t *max_u8, const uint8_t *q, uint8_t *s, uint8_t *levels, int B, int H,
                          int n_blocks, int n_max_blocks, float scale, hipStream_t st) {
    if constexpr (D <= 128) {
        // a block per wave, all its rows in flight at once (as in the fused step)
        dim3 grid((n_blocks + 3) / 4, H, B);
        hipLaunchKernelGGL((k_compute_cb64_kernel<D, REF, true>), grid, dim3(256), 0, st, f8, m4, l4, sum_u8, max_u8,
                           reinterpret_cast<const unsigned short *>(q), reinterpret_cast<unsigned short *>(s), levels,
                           n_blocks, n_max_blocks, H, 1, scale);
    } else {
        const int bpw = k_blocks_per_wave(B, H, n_blocks);
        dim3 grid((n_blocks + 4 * bpw - 1) / (4 * bpw), H, B);
        hipLaunchKernelGGL((k_compute_cb64_kernel<D, REF>), grid, dim3(256), 0, st, f8, m4, l4, sum_u8, max_u8,
                           reinterpret_cast<const unsigned short *>(q), reinterpret_cast<unsigned short *>(s), levels,
                           n_blocks, n_max_blocks, H, bpw, scale);
    }
}

template <int D, bool REF>
static void launch_k_cb256(const uint8_t *f8, const uint8_t *m4, const uint8_t *l4, const uint8_t *sum_u8,
                           const uint8_t *max_u8, const uint8_t *q, uint8_t *s, uint8_t *levels, int B, int H,
                           int n_blocks, int n_max_blocks, float scale, hipStream_t st) {
    const int bpw = k256_blocks_per_wave(B, H, n_blocks);
    dim3 grid((n_blocks + 4 * bpw - 1) / (4 * bpw), H, B);
    hipLaunchKernelGGL((k_compute_cb256_kernel<D, REF>), grid, dim3(256), 0, st, f8, m4, l4, sum_u8, max_u8,
                       reinterpret_cast<const unsigned short *>(q), reinterpret_cast<unsigned short *>(s), levels,
                       n_blocks, n_max_blocks, H, bpw, scale);
}

}  // namespace akv

using namespace akv;

namespace akv {
int launch_k_save_blocks(uint8_t *first_8, uint8_t *mid_4, uint8_t *last_4, const uint8_t *k_new, int bsz, int n_kv_heads,
                         int n_blocks, int n_max_blocks, int d_head, int d_block, int start_pos, int seqlen,
                         hipStream_t st) {
    AKV_REQUIRE(first_8 && mid_4 && last_4 && k_new, "k_cache_save: null pointer");
    AKV_REQUIRE(bsz > 0 && n_kv_heads > 0 && d_head > 0 && d_block > 0 && n_max_blocks > 0,
                "k_cache_save: non-positive dimension (bsz=%d heads=%d d_head=%d d_block=%d n_max_blocks=%d)", bsz,
                n_kv_heads, d_head, d_block, n_max_blocks);
    AKV_REQUIRE(d_block % 8 == 0 && d_head % 2 == 0, "k_cache_save: needs d_block %% 8 == 0 and even d_head (got %d, %d)",
                d_block, d_head);
    AKV_REQUIRE(start_pos >= 0 && seqlen >= 0 && n_blocks >= 0, "k_cache_save: negative start_pos/seqlen/n_blocks");
    AKV_REQUIRE(bsz <= 65535 && n_kv_heads <= 65535, "k_cache_save: bsz/heads exceed the grid limit 65535");
    const int tile_slots = d_block < 64 ? d_block : 64;
    // Beyond the reference: a run of whole 64-token tiles appended inside a larger block (d_block a multiple of
    // 64, start_pos and seqlen multiples of 64).  The reference launches nothing for this combination; the result
    // here is that of seqlen calls of its single-token branch (extension/csrc/K_cache.cu:63-94,142-162).
    const bool tile_append = start_pos != 0 && seqlen % d_block != 0 && seqlen > 1 && d_block % 64 == 0 &&
                             start_pos % 64 == 0 && seqlen % 64 == 0;
    if (start_pos == 0 || seqlen % d_block == 0 || tile_append) {
        if (n_blocks == 0) return AKV_OK;
        AKV_REQUIRE(start_pos % tile_slots == 0, "k_cache_save: start_pos=%d is not a multiple of %d", start_pos, tile_slots);
        // the reference's block branch stores the tokens of its first n_blocks blocks
        const int n_tokens = tile_append ? seqlen : (int)min((int64_t)seqlen, (int64_t)n_blocks * d_block);
        AKV_REQUIRE(tile_append || (int64_t)(n_blocks - 1) * d_block < seqlen, "k_cache_save: n_blocks=%d needs more than seqlen=%d tokens",
                    n_blocks, seqlen);
        AKV_REQUIRE(((int64_t)start_pos + n_tokens + d_block - 1) / d_block <= n_max_blocks,
                    "k_cache_save: tokens %d..%d exceed n_max_blocks=%d blocks of %d", start_pos, start_pos + n_tokens, n_max_blocks,
                    d_block);
        size_t lds = (size_t)tile_slots * (d_head + 2) * sizeof(unsigned short);
        AKV_REQUIRE(lds <= 64 * 1024, "k_cache_save: d_head=%d too large for the staging tile (%zu bytes)", d_head, lds);
        // whole tiles of 16-byte aligned data take the vector kernel (first tiles as long as divide the block, then of
        // 64 tokens), what remains the general one
        const bool vec = tile_slots == 64 && d_block % 64 == 0 && d_head % 8 == 0 && ((uintptr_t)k_new & 15) == 0 &&
                         (((uintptr_t)first_8 | (uintptr_t)mid_4 | (uintptr_t)last_4) & 7) == 0;
        const int n_tiles = (n_tokens + tile_slots - 1) / tile_slots;
        int n_vec = 0;       // 64-token tiles done by the vector kernel
        if (vec) {
            int done = 0;    // tokens
            const int big = d_block % 256 == 0 ? 256 : (d_block % 128 == 0 ? 128 : 64);
            for (int ts = big; ts >= 64; ts = ts > 64 ? 64 : 0) {
                if (ts != 64 && (start_pos + done) % ts != 0) continue;
                const int n = (n_tokens - done) / ts;
                if (n == 0) continue;
                // channels per workgroup: a divisor of d_head (in whole vectors) that keeps the tile within 32 KiB
                int dc = d_head;
                while (dc > 8 && (2 * ts * dc > 32 * 1024 || d_head % dc != 0 || dc % 8 != 0)) dc -= 8;
                if (2 * ts * dc > 64 * 1024) continue;
                const int threads = min(256, (ts * dc / 64 + 63) / 64 * 64);
                hipLaunchKernelGGL(k_save_tiles_kernel, dim3(n * (d_head / dc), n_kv_heads, bsz), dim3(threads), (size_t)2 * ts * dc, st,
                                   first_8, mid_4, last_4, reinterpret_cast<const u32x4 *>(k_new), n_max_blocks, n_kv_heads, d_head,
                                   d_block, ts, dc, start_pos, done, seqlen);
                int rc = check_launch("k_cache_save(tiles)");
                if (rc != AKV_OK) return rc;
                done += n * ts;
            }
            n_vec = done / 64;
        }
        if (n_tiles > n_vec) {
            hipLaunchKernelGGL(k_save_blocks_kernel, dim3(n_tiles - n_vec, n_kv_heads, bsz), dim3(256), lds, st, first_8, mid_4,
                               last_4, reinterpret_cast<const unsigned short *>(k_new), n_max_blocks, n_kv_heads, d_head,
                               d_block, tile_slots, start_pos, n_tokens, seqlen, n_vec);
            return check_launch("k_cache_save");
        }
        return AKV_OK;
    }
    if (seqlen == 1) {
        const int blk = start_pos / d_block;
        AKV_REQUIRE(blk < n_max_blocks, "k_cache_save: start_pos=%d beyond n_max_blocks=%d", start_pos, n_max_blocks);
        hipLaunchKernelGGL(k_save_token_kernel, dim3(n_kv_heads, bsz), dim3(d_head < 256 ? d_head : 256), 0, st,
                           first_8, mid_4, last_4, reinterpret_cast<const unsigned short *>(k_new), n_max_blocks,
                           n_kv_heads, d_head, d_block, blk, start_pos - blk * d_block);
        return check_launch("k_cache_save(token)");
    }
    // the reference launches nothing for this combination (extension/csrc/K_cache.cu:120,142)
    return AKV_OK;
}
}  // namespace akv

extern "C" int akv_k_cache_save(uint8_t *first_8, uint8_t *mid_4, uint8_t *last_4, const uint8_t *k_new, int bsz,
                                int n_kv_heads, int n_blocks, int n_max_blocks, int d_head, int d_block,
                                int start_pos, int seqlen, akv_stream_t stream) {
    return launch_k_save_blocks(first_8, mid_4, last_4, k_new, bsz, n_kv_heads, n_blocks, n_max_blocks, d_head, d_block,
                                start_pos, seqlen, static_cast<hipStream_t>(stream));
}

extern "C" int akv_k_cache_compute(const uint8_t *first_8, const uint8_t *mid_4, const uint8_t *last_4,
                                   const uint8_t *sum_u8, const uint8_t *max_u8, const uint8_t *q, uint8_t *s_out,
                                   uint8_t *levels_out, int bsz, int n_kv_heads, int n_blocks, int n_max_blocks,
                                   int d_head, int d_block, int seqlen, float sqrt_dim, int reference,
                                   akv_stream_t stream) {
    (void)seqlen;
    AKV_REQUIRE(first_8 && mid_4 && last_4 && q && s_out, "k_cache_compute: null pointer");
    AKV_REQUIRE(reference || (sum_u8 && max_u8), "k_cache_compute: null exponent-sum pointer");
    AKV_REQUIRE(bsz > 0 && n_kv_heads > 0 && d_head > 0 && d_block > 0 && n_max_blocks > 0 && n_blocks >= 0,
                "k_cache_compute: bad dimension (bsz=%d heads=%d d_head=%d d_block=%d n_blocks=%d n_max_blocks=%d)", bsz,
                n_kv_heads, d_head, d_block, n_blocks, n_max_blocks);
    AKV_REQUIRE(n_blocks <= n_max_blocks, "k_cache_compute: n_blocks=%d > n_max_blocks=%d", n_blocks, n_max_blocks);
    AKV_REQUIRE(d_block % 2 == 0 && d_block / 2 <= 1024, "k_cache_compute: d_block must be even and <= 2048");
    AKV_REQUIRE(bsz <= 65535 && n_kv_heads <= 65535, "k_cache_compute: bsz/heads exceed the grid limit 65535");
    AKV_REQUIRE((int64_t)n_max_blocks * d_head * d_block < (int64_t)1 << 31,
                "k_cache_compute: one (batch, head) slice of first_8 must stay below 2 GiB");
    if (n_blocks == 0) return AKV_OK;   // reference returns the uninitialised tensor, K_cache.cu:331-333
    hipStream_t st = static_cast<hipStream_t>(stream);
    // the reference multiplies by __float2half2_rn(sqrt_dim): the scale is rounded to fp16
    const float scale = __half2float(__float2half_rn(sqrt_dim));
    const bool ref = reference != 0;
#define AKV_K_TUNED(DD)                                                                                          \
    if (ref)                                                                                                     \
        launch_k_cb64<DD, true>(first_8, mid_4, last_4, sum_u8, max_u8, q, s_out, levels_out, bsz, n_kv_heads,   \
                                n_blocks, n_max_blocks, scale, st);                                              \
    else                                                                                                         \
        launch_k_cb64<DD, false>(first_8, mid_4, last_4, sum_u8, max_u8, q, s_out, levels_out, bsz, n_kv_heads,  \
                                 n_blocks, n_max_blocks, scale, st);
    if (d_block == 256 && (d_head == 128 || d_head == 64)) {
        if (d_head == 128) {
            if (ref) launch_k_cb256<128, true>(first_8, mid_4, last_4, sum_u8, max_u8, q, s_out, levels_out, bsz, n_kv_heads, n_blocks, n_max_blocks, scale, st);
            else launch_k_cb256<128, false>(first_8, mid_4, last_4, sum_u8, max_u8, q, s_out, levels_out, bsz, n_kv_heads, n_blocks, n_max_blocks, scale, st);
        } else {
            if (ref) launch_k_cb256<64, true>(first_8, mid_4, last_4, sum_u8, max_u8, q, s_out, levels_out, bsz, n_kv_heads, n_blocks, n_max_blocks, scale, st);
            else launch_k_cb256<64, false>(first_8, mid_4, last_4, sum_u8, max_u8, q, s_out, levels_out, bsz, n_kv_heads, n_blocks, n_max_blocks, scale, st);
        }
    } else if (d_block == 64 && d_head == 128) {
        AKV_K_TUNED(128)
    } else if (d_block == 64 && d_head == 64) {
        AKV_K_TUNED(64)
    } else if (d_block == 64 && d_head == 256) {
        AKV_K_TUNED(256)
    } else {
        dim3 grid(n_blocks, n_kv_heads, bsz), block(d_block / 2);
        if (ref)
            hipLaunchKernelGGL(k_compute_generic_kernel<true>, grid, block, 0, st, first_8, mid_4, last_4, sum_u8,
                               max_u8, reinterpret_cast<const unsigned short *>(q),
                               reinterpret_cast<unsigned short *>(s_out), levels_out, n_blocks, n_max_blocks,
                               n_kv_heads, d_head, d_block, scale);
        else
            hipLaunchKernelGGL(k_compute_generic_kernel<false>, grid, block, 0, st, first_8, mid_4, last_4, sum_u8,
                               max_u8, reinterpret_cast<const unsigned short *>(q),
                               reinterpret_cast<unsigned short *>(s_out), levels_out, n_blocks, n_max_blocks,
                               n_kv_heads, d_head, d_block, scale);
    }
#undef AKV_K_TUNED
    return check_launch("k_cache_compute");
}
