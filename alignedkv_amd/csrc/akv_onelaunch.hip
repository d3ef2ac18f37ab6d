// The fused decode step as ONE launch (multi-head caches of uniform length, head_dim 64 or 128).
//
// The multi-launch step leaves HBM idle between its kernels and while every (batch, head) row runs its middle stage
// (append, softmax, probe, threshold: a chain of dependent round trips during which a row reads almost nothing) at
// the same time.  Here a grid of resident workgroups walks through the whole step, and what has to wait for
// something else is picked up by whoever gets there last:
//
//   K items   a 256-token stretch of one row's K planes each (the work of one workgroup of the K-pass kernels), handed
//             out through a ticket counter in row order.  The workgroup that completes the last stretch of a row
//             (a counter per row) runs that row's middle stage on the spot -- while every other workgroup goes on
//             streaming K planes -- and publishes the row.
//   V items   a chunk of one published row's V planes each, handed out through a second ticket counter once the K
//             tickets have run out; partial sums per chunk, and the workgroup that completes a row's last chunk adds
//             them in a fixed order (the output bits do not depend on who finished when) and writes the row's output.
//
// Nobody waits for a workgroup that is not running: tickets are only ever held by running workgroups, so a row that a
// V ticket refers to is published after a bounded time by the workgroup that holds its last K stretch or runs its
// middle stage.  That wait polls with a limit; a waiter that hits the limit gives up, counts it in the control
// block (readable through akv_decode_step_timeouts) and leaves, so the kernel always ends.
// What one workgroup writes and another reads inside the launch (scores, probabilities, thresholds, partial sums, the
// counters) goes through device-scope accesses: the eight XCDs keep separate L2 caches.
#include "akv_step_parts.h"

#include <mutex>

namespace akv {

constexpr int kOneLaunchMaxRows = 4096;
constexpr int kOneLaunchSlots = 8;        // control blocks = streams (per device) that can use the one-launch step

// Counters of one step in flight.  All zero between steps: the last workgroup to leave a step clears what the step
// used (`timeouts` is never cleared by the device).
struct StepCtl {
    u32 kticket, vticket, n_published, exited;
    u32 timeouts;
    u32 pad[11];
    u32 kdone[kOneLaunchMaxRows];       // K stretches of the row completed
    u32 vdone[kOneLaunchMaxRows];       // V chunks of the row completed
    u32 published[kOneLaunchMaxRows];   // [slot]: row + 1 of the slot-th row whose middle stage is done (0: not yet)
};
static __device__ __align__(256) StepCtl g_step_ctl[kOneLaunchSlots];

__device__ __forceinline__ u32 ctl_add(u32 *p, u32 v) {
    return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ u32 ctl_load(u32 *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void ctl_store(u32 *p, u32 v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// Workgroup barrier that first waits until every memory operation of the wave has completed: the device-scope stores
// issued before it have reached the point where every XCD sees them.
__device__ __forceinline__ void barrier_after_stores() {
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

#ifdef AKV_TRACE
// Development aid (not compiled into the library): per workgroup, timestamps of the phases of one step.
static unsigned long long *g_trace_buffer = nullptr;
#define AKV_TRACE_MARK(i) do { if (a.trace != nullptr && tid == 0) a.trace[(size_t)blockIdx.x * 16 + (i)] = __builtin_amdgcn_s_memrealtime(); } while (0)
#define AKV_TRACE_ADD(i, v) do { if (a.trace != nullptr && tid == 0) a.trace[(size_t)blockIdx.x * 16 + (i)] += (v); } while (0)
#else
#define AKV_TRACE_MARK(i) do { } while (0)
#define AKV_TRACE_ADD(i, v) do { } while (0)
#endif

struct OneLaunchArgs {
    const uint8_t *k_first_8, *k_mid_4, *k_last_4;
    const uint8_t *v_first_8, *v_mid_4, *v_last_4;
    MiddleArgs ma;
    float *partial;
    unsigned short *out;
    uint8_t *k_levels_out, *v_levels_out, *amin_out;
    StepCtl *ctl;
    float scale;
    int rows;          // (batch, head) pairs
    int R;             // flushed tokens of every row once this step's token is appended
    int nkc;           // K items per row (stretches of 256 tokens)
    int nvc;           // V items per row (chunks of 4 * tokens_per_wave tokens)
    int spin_limit;    // polls a waiter spends on one row before it gives up
#ifdef AKV_TRACE
    unsigned long long *trace;
#endif
};

// grid: resident workgroups (a few per compute unit), 256 threads.  KB: tokens per K plane block (64 or 256).
template <int D, bool REF, int KB, int NIT>
__global__ __launch_bounds__(256) void one_launch_step_kernel(const OneLaunchArgs a) {
    constexpr int TPW = (D == 256 ? 32 : 64) * NIT;   // tokens per wave and V item
    constexpr int CT = 4 * TPW;                        // tokens per V item
    __shared__ u32 sh_item, sh_done, sh_row;
    __shared__ float wave_part[4][D];
    const int tid = threadIdx.x;
    StepCtl *ctl = a.ctl;
    const StepGeom &geo = a.ma.g;
    const int R = a.R;

    // ---- K items ------------------------------------------------------------------------------------------------
    const u32 n_kitems = (u32)a.rows * (u32)a.nkc;
    AKV_TRACE_MARK(0);
    if (tid == 0) sh_item = ctl_add(&ctl->kticket, 1u);
    __syncthreads();
    u32 item = sh_item;
    AKV_TRACE_MARK(1);
    while (item < n_kitems) {
        AKV_TRACE_ADD(8, 1);
        const int row = (int)(item / (u32)a.nkc), stretch = (int)(item - (u32)row * (u32)a.nkc);
        if constexpr (KB == 256)
            k_pass256_split_block<D, REF, 4>(a.k_first_8, a.k_mid_4, a.k_last_4, a.ma.kcm, a.ma.q, a.ma.k_new, a.ma.scores,
                                             a.k_levels_out, geo, a.scale, stretch, row, R);
        else
            k_pass64_whole_blocks<D, REF>(a.k_first_8, a.k_mid_4, a.k_last_4, a.ma.kcm, a.ma.q, a.ma.k_new, a.ma.scores,
                                          a.k_levels_out, geo, a.scale, stretch, row, row, R);
#ifdef AKV_TRACE
        const unsigned long long t_k0 = __builtin_amdgcn_s_memrealtime();
#endif
        barrier_after_stores();
#ifdef AKV_TRACE
        const unsigned long long t_k1 = __builtin_amdgcn_s_memrealtime();
        AKV_TRACE_ADD(10, t_k1 - t_k0);
#endif
        if (tid == 0) {
            // the row's counter and the next ticket in one round trip
            const u32 done = ctl_add(&ctl->kdone[row], 1u), next = ctl_add(&ctl->kticket, 1u);
            sh_done = done;
            sh_item = next;
        }
        __syncthreads();
#ifdef AKV_TRACE
        AKV_TRACE_ADD(11, __builtin_amdgcn_s_memrealtime() - t_k1);
#endif
        const bool last_of_row = sh_done == (u32)a.nkc - 1u;
        item = sh_item;
        if (last_of_row) {
            AKV_TRACE_ADD(9, 1);
            // every stretch of the row has its scores in memory: append, softmax, probe, threshold, tail output
            middle_body<D, 256, NoHook, true>(a.ma, row);
            barrier_after_stores();
            if (tid == 0) {
                const u32 slot = ctl_add(&ctl->n_published, 1u);
                ctl_store(&ctl->published[slot], (u32)row + 1u);
            }
        }
    }

    // ---- V items ------------------------------------------------------------------------------------------------
    const u32 n_vitems = (u32)a.rows * (u32)a.nvc;
    __syncthreads();
    AKV_TRACE_MARK(2);
    if (tid == 0) sh_item = ctl_add(&ctl->vticket, 1u);
    __syncthreads();
    item = sh_item;
    AKV_TRACE_MARK(3);
    while (item < n_vitems) {
        AKV_TRACE_ADD(12, 1);
#ifdef AKV_TRACE
        const unsigned long long t_v0 = __builtin_amdgcn_s_memrealtime();
#endif
        u32 next = 0;
        if (tid == 0) next = ctl_add(&ctl->vticket, 1u);
        const int slot = (int)(item / (u32)a.nvc), chunk = (int)(item - (u32)slot * (u32)a.nvc);
        if (tid == 0) {
            u32 v = ctl_load(&ctl->published[slot]);
            for (int spins = 0; v == 0u && spins < a.spin_limit; ++spins) {
                __builtin_amdgcn_s_sleep(32);
                v = ctl_load(&ctl->published[slot]);
            }
            if (v == 0u) ctl_add(&ctl->timeouts, 1u);
            sh_row = v;
            sh_item = next;
        }
        __syncthreads();
#ifdef AKV_TRACE
        const unsigned long long t_v1 = __builtin_amdgcn_s_memrealtime();
        AKV_TRACE_ADD(13, t_v1 - t_v0);
#endif
        const u32 pub = sh_row;
        item = sh_item;
        if (pub == 0u) {             // gave up on this row (counted); the step's output is then incomplete
            __syncthreads();         // (everybody has read the shared words before thread 0 overwrites them)
            continue;
        }
        const int row = (int)pub - 1;
        const int wave = wave_index();
        const int t_begin = (chunk * 4 + wave) * TPW;
        const int t_end = min(t_begin + TPW, R);
        const int64_t row0 = (int64_t)row * geo.max_seq_len;
        VFirstTile<D> ft;
        v_prefetch_first<D>(ft, a.v_first_8 + row0 * D, R, t_begin, t_end);
        const unsigned char amin = REF ? 0 : (unsigned char)__builtin_amdgcn_raw_buffer_load_b8(make_rsrc(a.ma.amin + row, 1u), 0, 0, kDeviceScope);
        if (!REF && a.amin_out != nullptr && chunk == 0 && tid == 0) a.amin_out[row] = amin;
        float acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
        v_accumulate<D, REF, NIT, kDeviceScope>(ft, a.v_first_8 + row0 * D, a.v_mid_4 + row0 * (D / 2), a.v_last_4 + row0 * (D / 2), R,
                                                a.ma.probs + (int64_t)row * geo.row_stride, amin, t_begin, t_end, acc,
                                                a.v_levels_out != nullptr ? a.v_levels_out + (int64_t)row * R : nullptr);
        v_fold_workgroup<D>(acc, wave_part, a.partial + ((int64_t)row * a.nvc + chunk) * D);
        barrier_after_stores();
#ifdef AKV_TRACE
        const unsigned long long t_v2 = __builtin_amdgcn_s_memrealtime();
        AKV_TRACE_ADD(14, t_v2 - t_v1);
#endif
        if (tid == 0) sh_done = ctl_add(&ctl->vdone[row], 1u);
        __syncthreads();
#ifdef AKV_TRACE
        AKV_TRACE_ADD(15, __builtin_amdgcn_s_memrealtime() - t_v2);
#endif
        if (sh_done == (u32)a.nvc - 1u) {
            // the row's last chunk: out = fp16(fp16(sum of the chunks in their fixed order) + tail), the fp16 `o += tail`
            // of the reference (extension/v_cache_file.py:189)
            const __amdgpu_buffer_rsrc_t rP = make_rsrc(a.partial + (int64_t)row * a.nvc * D, (u32)a.nvc * D * 4);
            const __amdgpu_buffer_rsrc_t rT = make_rsrc(a.ma.otail + (int64_t)row * D, (u32)D * 2);
            for (int d = tid; d < D; d += 256) {
                float sum = 0.f;
                int c = 0;
                for (; c + 8 <= a.nvc; c += 8) {
                    float v[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) v[i] = load_f32_device(rP, ((c + i) * D + d) * 4);
#pragma unroll
                    for (int i = 0; i < 8; ++i) sum += v[i];
                }
                for (; c < a.nvc; ++c) sum += load_f32_device(rP, (c * D + d) * 4);
                const float o16 = half_bits_to_float(float_to_half_bits(sum));
                const u32 tail = (u32)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(rT, d * 2, 0, kDeviceScope);
                a.out[(int64_t)row * D + d] = float_to_half_bits(o16 + half_bits_to_float(tail));
            }
        }
    }

    // ---- leave: the last workgroup out clears the counters for the next step ------------------------------------------
    __syncthreads();
    AKV_TRACE_MARK(4);
    if (tid == 0) sh_done = ctl_add(&ctl->exited, 1u);
    __syncthreads();
    if (sh_done == gridDim.x - 1u) {
        for (int r = tid; r < a.rows; r += 256) {
            ctl_store(&ctl->kdone[r], 0u);
            ctl_store(&ctl->vdone[r], 0u);
            ctl_store(&ctl->published[r], 0u);
        }
        if (tid == 0) {
            ctl_store(&ctl->kticket, 0u);
            ctl_store(&ctl->vticket, 0u);
            ctl_store(&ctl->n_published, 0u);
            ctl_store(&ctl->exited, 0u);
        }
    }
}

// ---- host side ------------------------------------------------------------------------------------------------------
namespace {
constexpr int kMaxDevices = 64;
std::mutex g_ctl_mutex;
StepCtl *g_ctl_base[kMaxDevices];                 // per device: address of that device's g_step_ctl
struct SlotOwner {
    bool used;
    hipStream_t stream;
};
SlotOwner g_slot_owner[kMaxDevices][kOneLaunchSlots];

// Control block of (current device, stream); null when the device has run out of blocks (or on an error, with `rc` set).
StepCtl *control_block(hipStream_t st, int &rc) {
    rc = AKV_OK;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(g_ctl_mutex);
    if (g_ctl_base[dev] == nullptr) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_step_ctl));
        if (e != hipSuccess || p == nullptr) {
            set_error("decode_step: hipGetSymbolAddress(control blocks) failed on device %d: %s", dev, hipGetErrorString(e));
            rc = AKV_ERR_LAUNCH;
            return nullptr;
        }
        g_ctl_base[dev] = static_cast<StepCtl *>(p);
    }
    SlotOwner *own = g_slot_owner[dev];
    for (int i = 0; i < kOneLaunchSlots; ++i)
        if (own[i].used && own[i].stream == st) return g_ctl_base[dev] + i;
    for (int i = 0; i < kOneLaunchSlots; ++i)
        if (!own[i].used) {
            own[i].used = true;
            own[i].stream = st;
            return g_ctl_base[dev] + i;
        }
    return nullptr;
}
}  // namespace

// Whether the one-launch step covers this shape (the caller has checked: one query head per KV head, one length for all
// sequences, threshold indexing not literal).
bool one_launch_covers(int D, int kb, int rows, int R) {
    return (D == 64 || D == 128) && (kb == 64 || kb == 256) && rows <= kOneLaunchMaxRows && R >= 64;
}

// Launches the step; AKV_OK + *launched = false when no control block is free for this stream (the caller then takes the
// multi-launch path).
template <int D>
int launch_one_launch_step(const uint8_t *kf8, const uint8_t *km4, const uint8_t *kl4, const uint8_t *vf8, const uint8_t *vm4,
                           const uint8_t *vl4, const MiddleArgs &ma, float *partial, unsigned short *out, uint8_t *k_levels_out,
                           uint8_t *v_levels_out, uint8_t *amin_out, int rows, int R, int kb, bool ref, float scale,
                           hipStream_t st, bool *launched) {
    *launched = false;
    int rc = AKV_OK;
    StepCtl *ctl = control_block(st, rc);
    if (ctl == nullptr) return rc;
    constexpr int NIT = 1;
    constexpr int CT = 4 * (D == 256 ? 32 : 64) * NIT;
    OneLaunchArgs a;
    a.k_first_8 = kf8; a.k_mid_4 = km4; a.k_last_4 = kl4;
    a.v_first_8 = vf8; a.v_mid_4 = vm4; a.v_last_4 = vl4;
    a.ma = ma;
    a.partial = partial;
    a.out = out;
    a.k_levels_out = k_levels_out; a.v_levels_out = v_levels_out; a.amin_out = amin_out;
    a.ctl = ctl;
    a.scale = scale;
    a.rows = rows;
    a.R = R;
    a.nkc = (R + 255) / 256;
    a.nvc = (R + CT - 1) / CT;
#ifdef AKV_TRACE
    a.trace = g_trace_buffer;
#endif
    a.spin_limit = 1 << 20;
    { AKV_TUNE("AKV_TUNE_SPIN_LIMIT", v); if (has_v) a.spin_limit = v < 0 ? 0 : v; }
    int per_cu = 4;
    { AKV_TUNE("AKV_TUNE_WG_PER_CU", v); if (has_v && v > 0) per_cu = v; }
    const int cus = compute_units() > 0 ? compute_units() : 256;
    const int64_t most = (int64_t)rows * (a.nkc > a.nvc ? a.nkc : a.nvc);
    const int grid = (int)(most < (int64_t)cus * per_cu ? most : (int64_t)cus * per_cu);
#define AKV_ONE(RF, KBV) hipLaunchKernelGGL((one_launch_step_kernel<D, RF, KBV, NIT>), dim3(grid), dim3(256), 0, st, a)
    if (kb == 256) {
        if (ref) AKV_ONE(true, 256); else AKV_ONE(false, 256);
    } else {
        if (ref) AKV_ONE(true, 64); else AKV_ONE(false, 64);
    }
#undef AKV_ONE
    *launched = true;
    return check_launch("decode_step(one launch)");
}

template int launch_one_launch_step<64>(const uint8_t *, const uint8_t *, const uint8_t *, const uint8_t *, const uint8_t *,
                                        const uint8_t *, const MiddleArgs &, float *, unsigned short *, uint8_t *, uint8_t *,
                                        uint8_t *, int, int, int, bool, float, hipStream_t, bool *);
template int launch_one_launch_step<128>(const uint8_t *, const uint8_t *, const uint8_t *, const uint8_t *, const uint8_t *,
                                         const uint8_t *, const MiddleArgs &, float *, unsigned short *, uint8_t *, uint8_t *,
                                         uint8_t *, int, int, int, bool, float, hipStream_t, bool *);

}  // namespace akv

using namespace akv;

extern "C" int akv_decode_step_timeouts(akv_stream_t stream, unsigned int *timeouts) {
    AKV_REQUIRE(timeouts != nullptr, "decode_step_timeouts: null pointer");
    *timeouts = 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error("decode_step_timeouts: no current device");
        return AKV_ERR_LAUNCH;
    }
    StepCtl *ctl = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_ctl_mutex);
        if (g_ctl_base[dev] != nullptr)
            for (int i = 0; i < kOneLaunchSlots; ++i)
                if (g_slot_owner[dev][i].used && g_slot_owner[dev][i].stream == st) ctl = g_ctl_base[dev] + i;
    }
    if (ctl == nullptr) return AKV_OK;     // this stream never ran the one-launch step
    if (hipStreamSynchronize(st) != hipSuccess ||
        hipMemcpy(timeouts, &ctl->timeouts, sizeof(unsigned int), hipMemcpyDeviceToHost) != hipSuccess) {
        set_error("decode_step_timeouts: reading the control block failed");
        return AKV_ERR_LAUNCH;
    }
    return AKV_OK;
}

#ifdef AKV_TRACE
extern "C" __attribute__((visibility("default"))) void akv_debug_trace_buffer(void *p) { g_trace_buffer = static_cast<unsigned long long *>(p); }
#endif
