// Shared device helpers of the AlignedKV HIP kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "../../include/alignedkv.h"

typedef uint32_t u32;
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));

namespace akv {

// ---- host-side error reporting -------------------------------------------------------------
void set_error(const char *fmt, ...);
int check_launch(const char *what);
int compute_units();   // of the current device (0: unknown)

// Tuning switches from the environment (AKV_TUNE_*), read once per call site and again after
// akv_reload_tuning(): a getenv per switch and step costs a few microseconds of host time per decode step,
// which is what a batch-1 step is bound by.
extern int g_tune_epoch;
struct TuneVar {
    const char *name;
    int epoch;
    bool present;
    int value;
    bool get(int &out) {
        if (epoch != g_tune_epoch) {
            const char *e = getenv(name);
            present = e != nullptr;
            value = e != nullptr ? atoi(e) : 0;
            epoch = g_tune_epoch;
        }
        out = value;
        return present;
    }
};
#define AKV_TUNE(NAME, VAR) static akv::TuneVar tune_##VAR = {NAME, -1, false, 0}; int VAR = 0; const bool has_##VAR = tune_##VAR.get(VAR)

#define AKV_REQUIRE(cond, ...)            \
    do {                                   \
        if (!(cond)) {                     \
            akv::set_error(__VA_ARGS__);   \
            return AKV_ERR_INVALID;        \
        }                                  \
    } while (0)

// ---- fp16 bit helpers ------------------------------------------------------------------------
__device__ __forceinline__ float half_bits_to_float(u32 bits16) {
    return __half2float(__ushort_as_half((unsigned short)bits16));
}
__device__ __forceinline__ float lo_half_to_float(u32 w) {
    return __half2float(__ushort_as_half((unsigned short)(w & 0xffffu)));
}
__device__ __forceinline__ float hi_half_to_float(u32 w) {
    return __half2float(__ushort_as_half((unsigned short)(w >> 16)));
}
__device__ __forceinline__ unsigned short float_to_half_bits(float f) {
    return __half_as_ushort(__float2half_rn(f));
}

// ---- fetch levels ------------------------------------------------------------------------------
// K: per (batch, head, channel); diff is computed in uint8 (reference: extension/csrc/K_cache.cu:211,249-250).
__device__ __forceinline__ int k_level(unsigned char max_u8, unsigned char sum_u8) {
    unsigned char diff = (unsigned char)(max_u8 - sum_u8);
    return diff >= 8 ? 2 : (diff >= 4 ? 1 : 0);
}
// V: per (batch, head, token); `amin << 10` and the difference live in 16-bit signed integers
// (reference: extension/csrc/V_cache.cu:195-197,211,250-251).
__device__ __forceinline__ int v_level(unsigned char amin_u8, unsigned short s_bits) {
    short a = (short)((unsigned short)((unsigned)amin_u8 << 10));
    short diff = (short)((unsigned short)((unsigned short)a - s_bits));
    return diff >= 0x0800 ? 2 : (diff >= 0x0400 ? 1 : 0);
}

// ---- 8 elements at a time ------------------------------------------------------------------------
// Ha/Hb: high bytes of elements 0..3 / 4..7; M, L: the 4 mid / last bytes covering the same 8
// elements (even element in the high nibble).  Skipped planes are passed as the substitution
// bytes (M = 0x88888888, L = 0 for level 2; L = 0x88888888 for level 1), which reproduces
// hi<<8|0x80 and hi<<8|mid<<4|0x8 (reference: extension/csrc/K_cache.cu:201-205,249-252).
// acc[i] += value(element i) * x.
// E / O: the low bytes of the even / odd elements of 8 elements, from their 4 mid and 4 last bytes.
__device__ __forceinline__ void split_even_odd(u32 M, u32 L, u32 &E, u32 &O) {
    E = (M & 0xF0F0F0F0u) | ((L >> 4) & 0x0F0F0F0Fu);   // low bytes of elements 0,2,4,6
    O = ((M << 4) & 0xF0F0F0F0u) | (L & 0x0F0F0F0Fu);   // low bytes of elements 1,3,5,7
}
__device__ __forceinline__ void fma8_even_odd(float *acc, u32 Ha, u32 Hb, u32 E, u32 O, float x) {
    u32 w02 = __builtin_amdgcn_perm(Ha, E, 0x06010400u);
    u32 w13 = __builtin_amdgcn_perm(Ha, O, 0x07010500u);
    u32 w46 = __builtin_amdgcn_perm(Hb, E, 0x06030402u);
    u32 w57 = __builtin_amdgcn_perm(Hb, O, 0x07030502u);
    acc[0] = fmaf(lo_half_to_float(w02), x, acc[0]);
    acc[2] = fmaf(hi_half_to_float(w02), x, acc[2]);
    acc[1] = fmaf(lo_half_to_float(w13), x, acc[1]);
    acc[3] = fmaf(hi_half_to_float(w13), x, acc[3]);
    acc[4] = fmaf(lo_half_to_float(w46), x, acc[4]);
    acc[6] = fmaf(hi_half_to_float(w46), x, acc[6]);
    acc[5] = fmaf(lo_half_to_float(w57), x, acc[5]);
    acc[7] = fmaf(hi_half_to_float(w57), x, acc[7]);
}
__device__ __forceinline__ void fma8(float *acc, u32 Ha, u32 Hb, u32 M, u32 L, float x) {
    u32 E, O;
    split_even_odd(M, L, E, O);
    fma8_even_odd(acc, Ha, Hb, E, O, x);
}
// A fetch level as a pair (keep, put) applied to the even/odd low bytes of fully fetched planes:
// low = (low & keep) | put gives low (level 0), (mid << 4) | 0x8 (level 1), 0x80 (level 2).  Used where
// several query heads with different levels share one fetched tile.
__device__ __forceinline__ void level_masks(int level, u32 &keep, u32 &put) {
    keep = level == 0 ? 0xFFFFFFFFu : (level == 1 ? 0xF0F0F0F0u : 0u);
    put = level == 0 ? 0u : (level == 1 ? 0x08080808u : 0x80808080u);
}

// Scalar reconstruction used by the generic (any-shape) kernels.
__device__ __forceinline__ u32 rebuild_bits(u32 hi, u32 mid_nibble, u32 last_nibble, int level) {
    u32 lo = level == 0 ? ((mid_nibble << 4) | last_nibble) : (level == 1 ? ((mid_nibble << 4) | 0x8u) : 0x80u);
    return (hi << 8) | lo;
}

// ---- buffer resources: loads whose byte offset is >= num_records return 0 and fetch nothing ---
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, u32 num_bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)num_bytes, 0x00020000);
}
// x / d for many x and one d: r = 1 / d once (a correctly rounded division), then per x a product and one
// correction step, three instructions instead of the ten of a division.  The result equals x / d as the division
// instruction sequence rounds it (checked on the host for 2e7 pairs with x in (0, 1], d in [1, 4096]); values too small
// for fp16 are not looked at by the callers.
__device__ __forceinline__ float div_by(float x, float d, float r) {
    const float q = x * r;
    return fmaf(fmaf(-q, d, x), r, q);
}

// exp(x) for x <= 0 (a score minus the row maximum): the hardware's 2^y on y = x * log2(e), with the product's rounding
// error and the low part of log2(e) put back as a first-order correction, so the result is within an ulp or two of the
// correctly rounded one for every x whose exponential is a normal float; below that it goes to zero (a probability
// that small rounds to zero in fp16 anyway).  Six instructions against the thirteen of the library routine, which
// matters where a compute unit runs a whole row's softmax on its own.
__device__ __forceinline__ float exp_nonpositive(float x) {
    const float l2e_hi = 1.44269502162933349609375f, l2e_lo = 1.925963033500011e-8f, ln2 = 0.693147182464599609375f;
    x = fmaxf(x, -200.f);      // (minus infinity, a masked score, included: the result is zero)
    const float y = x * l2e_hi;
    float err = fmaf(x, l2e_hi, -y);
    err = fmaf(x, l2e_lo, err);
    const float e = __builtin_amdgcn_exp2f(y);
    return fmaf(e, err * ln2, e);
}

// Makes the compiler fetch kernel arguments where this stands (the entry block) instead of in the block of their first
// use: arguments that are first needed behind a branch otherwise arrive in a scalar load of their own there, a
// dependent round trip in front of the loads that need them.  Only for kernels that look nothing up through uniform
// loads afterwards (task maps, per-sequence lengths): behind this statement the compiler no longer proves such loads
// unclobbered and issues them as vector loads.
template <typename... T>
__device__ __forceinline__ void fetch_arguments_now(T... p) {
    (..., [](auto x) { asm volatile("" ::"s"(x)); }(p));
}

constexpr int kSkip = 0x7fffffff;   // an offset no plane slice reaches

// Cache-policy bits of buffer loads/stores on gfx950: sc1 = device (agent) scope.  Data that one
// workgroup writes and another workgroup of the SAME launch reads (scores, partial sums) goes through
// these: the eight XCDs have separate L2 caches that are only reconciled at kernel boundaries, and a
// device-wide fence (write back + invalidate of a whole L2) costs far more than the few bytes exchanged.
constexpr int kDeviceScope = 1 << 4;
// Plane bytes are read once per step: non-temporal loads (they do not displace what the compute unit's cache holds
// and are not kept in it).  Measured on the V planes at batch 8 x 32 heads x 4096 tokens: 25.2 instead of 26.8 us.
constexpr int kStream = 1 << 1;
__device__ __forceinline__ void store_u16_device(const __amdgpu_buffer_rsrc_t r, int byte_off, unsigned short v) {
    __builtin_amdgcn_raw_buffer_store_b16((short)v, r, byte_off, 0, kDeviceScope);
}
// A score of the K pass, read by a later kernel.  through: written through to memory at once; otherwise it stays in L2
// until the kernel ends (cheaper while the scores of a launch are few: the wave's store is acknowledged sooner and the
// write-back of a few dirty lines at the kernel's end costs less than writing next to the streaming reads).
__device__ __forceinline__ void store_score(const __amdgpu_buffer_rsrc_t r, int byte_off, unsigned short v, bool through) {
    if (through) __builtin_amdgcn_raw_buffer_store_b16((short)v, r, byte_off, 0, kDeviceScope);
    else __builtin_amdgcn_raw_buffer_store_b16((short)v, r, byte_off, 0, 0);
}
__device__ __forceinline__ void store_f32_device(const __amdgpu_buffer_rsrc_t r, int byte_off, float v) {
    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), r, byte_off, 0, kDeviceScope);
}
__device__ __forceinline__ u32x4 load_b128_device(const __amdgpu_buffer_rsrc_t r, int byte_off) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, kDeviceScope);
}

// Index of the wave in its workgroup as a scalar: what is derived from it (a wave's share of the tokens, loop bounds,
// validity of a tile) then lives in scalar registers, loops over it are uniform loops and the conditions cost no
// vector instructions.  (threadIdx.x >> 6 alone is a per-lane value to the compiler.)
__device__ __forceinline__ int wave_index() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

// Wave-wide reductions with the result in every lane: two quad permutes and the two mirrors inside the 16-lane rows
// (data-parallel primitives: no LDS round trip per step, unlike a shuffle), then the four row totals through scalar
// registers.  The order of the additions is fixed, so the bits of a sum are reproducible.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
template <int CTRL>
__device__ __forceinline__ u32 dpp_u32(u32 v) {
    return (u32)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
}
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppHalfMirror = 0x141, kDppMirror = 0x140;
__device__ __forceinline__ float rows_to_wave_f32(float v, bool is_max) {
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return is_max ? fmaxf(fmaxf(r0, r1), fmaxf(r2, r3)) : (r0 + r1) + (r2 + r3);
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f32<kDppXor1>(v);
    v += dpp_f32<kDppXor2>(v);
    v += dpp_f32<kDppHalfMirror>(v);
    v += dpp_f32<kDppMirror>(v);
    return rows_to_wave_f32(v, false);
}
// Sum over groups of N consecutive lanes (N = 2, 4, 8 or 16, aligned): every lane of a group ends up with the group's
// sum, added in the order of a butterfly over lane distances 1, 2, 4, 8 (the mirrors pair the same partial sums as
// those distances do).
template <int N>
__device__ __forceinline__ float lane_group_sum(float v) {
    static_assert(N == 1 || N == 2 || N == 4 || N == 8 || N == 16, "a group lies inside a 16-lane row");
    if constexpr (N >= 2) v += dpp_f32<kDppXor1>(v);
    if constexpr (N >= 4) v += dpp_f32<kDppXor2>(v);
    if constexpr (N >= 8) v += dpp_f32<kDppHalfMirror>(v);
    if constexpr (N >= 16) v += dpp_f32<kDppMirror>(v);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_f32<kDppXor1>(v));
    v = fmaxf(v, dpp_f32<kDppXor2>(v));
    v = fmaxf(v, dpp_f32<kDppHalfMirror>(v));
    v = fmaxf(v, dpp_f32<kDppMirror>(v));
    return rows_to_wave_f32(v, true);
}
__device__ __forceinline__ u32 wave_min_u32(u32 v) {
    v = min(v, dpp_u32<kDppXor1>(v));
    v = min(v, dpp_u32<kDppXor2>(v));
    v = min(v, dpp_u32<kDppHalfMirror>(v));
    v = min(v, dpp_u32<kDppMirror>(v));
    return min(min((u32)__builtin_amdgcn_readlane((int)v, 0), (u32)__builtin_amdgcn_readlane((int)v, 16)),
               min((u32)__builtin_amdgcn_readlane((int)v, 32), (u32)__builtin_amdgcn_readlane((int)v, 48)));
}
// Maximum over the wave of a value that every lane of a 16-lane row holds alike: four lane reads, a scalar result.
__device__ __forceinline__ u32 rows_max_u32(u32 v) {
    return max(max((u32)__builtin_amdgcn_readlane((int)v, 0), (u32)__builtin_amdgcn_readlane((int)v, 16)),
               max((u32)__builtin_amdgcn_readlane((int)v, 32), (u32)__builtin_amdgcn_readlane((int)v, 48)));
}
// Maximum over the wave of a value that the lanes 4k .. 4k + 3 hold alike: two row rotations, then the rows.
__device__ __forceinline__ u32 quads_max_u32(u32 v) {
    v = max(v, (u32)__builtin_amdgcn_update_dpp(0, (int)v, 0x124, 0xf, 0xf, false));   // row_ror:4
    v = max(v, (u32)__builtin_amdgcn_update_dpp(0, (int)v, 0x128, 0xf, 0xf, false));   // row_ror:8
    return rows_max_u32(v);
}
__device__ __forceinline__ u32 wave_max_u32(u32 v) {
    v = max(v, dpp_u32<kDppXor1>(v));
    v = max(v, dpp_u32<kDppXor2>(v));
    v = max(v, dpp_u32<kDppHalfMirror>(v));
    v = max(v, dpp_u32<kDppMirror>(v));
    return rows_max_u32(v);
}
__device__ __forceinline__ int wave_sum_i32(int v) {
    v += (int)dpp_u32<kDppXor1>((u32)v);
    v += (int)dpp_u32<kDppXor2>((u32)v);
    v += (int)dpp_u32<kDppHalfMirror>((u32)v);
    v += (int)dpp_u32<kDppMirror>((u32)v);
    return (__builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16)) +
           (__builtin_amdgcn_readlane(v, 32) + __builtin_amdgcn_readlane(v, 48));
}


}  // namespace akv
