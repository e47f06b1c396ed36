// Shared device/host helpers for the gfx950 kernels.  Wave size is 64 everywhere.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include "../../include/rwkv_hip.h"

#define WAVE 64

typedef _Float16 h16;
typedef _Float16 h16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 h16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 h16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define DEV __device__ __forceinline__

// ---- launch bookkeeping -------------------------------------------------------------------
#define RWKV_LAUNCH_CHECK()                         \
    do {                                            \
        hipError_t e__ = hipGetLastError();         \
        if (e__ != hipSuccess) return (int)e__;     \
    } while (0)

static inline bool aligned16(const void *p) { return (((uintptr_t)p) & 15) == 0; }

// ---- fp16 <-> fp32 -----------------------------------------------------------------------
DEV float h2f(rwkv_half v) { return (float)__builtin_bit_cast(h16, v); }
DEV rwkv_half f2h(float v) { return __builtin_bit_cast(rwkv_half, (h16)v); }  // round-to-nearest-even
DEV float round_h(float v) { return (float)(h16)v; }

// ---- wave / block reductions ---------------------------------------------------------------
// Sums use DPP lane permutes (one VALU issue each, no LDS traffic): a butterfly inside each row
// of 16 lanes (xor 1, xor 2, half-mirror, mirror), then the four row totals are combined
// through v_readlane.  Every lane gets the result.
template <int CTRL>
DEV float dpp_mov(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
DEV float row16_sum(float v) {
    v += dpp_mov<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_mov<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_mov<0x141>(v);  // row_half_mirror
    v += dpp_mov<0x140>(v);  // row_mirror
    return v;
}
DEV float wave_sum(float v) {
    v = row16_sum(v);
    const int b = __builtin_bit_cast(int, v);
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
    const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
    const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
    return (r0 + r1) + (r2 + r3);
}
DEV float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}
DEV float wave_min(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, WAVE));
    return v;
}

// Sum over the whole workgroup; every thread gets the result.  `red` is LDS scratch of at
// least (blockDim.x / 64) floats; safe to call repeatedly with the same scratch.
DEV float block_sum(float v, float *red) {
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) red[wid] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += red[i];
    return t;
}

// Sum K values over the workgroup at once (one pair of barriers); every thread gets all K totals, each formed
// exactly as block_sum forms it.  `red` is LDS scratch of at least K * (blockDim.x / 64) floats.
template <int K>
DEV void block_sum_n(float (&v)[K], float *red) {
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = wave_sum(v[k]);
    __syncthreads();
    if (lane == 0)
#pragma unroll
        for (int k = 0; k < K; ++k) red[k * nw + wid] = v[k];
    __syncthreads();
#pragma unroll
    for (int k = 0; k < K; ++k) {
        float t = 0.f;
        for (int i = 0; i < nw; ++i) t += red[k * nw + i];
        v[k] = t;
    }
}

// ---- uint8 -> fp16 pairs -------------------------------------------------------------------
// Bytes b0..b3 of `v` become the fp16 values (1024 + b): placing a byte under the exponent
// byte 0x64 yields exactly 1024 + b.  lo = (b0, b1), hi = (b2, b3).
DEV h16x2 u8pair_lo_1024(uint32_t v) {
    return __builtin_bit_cast(h16x2, __builtin_amdgcn_perm(0x64646464u, v, 0x05010400u));
}
DEV h16x2 u8pair_hi_1024(uint32_t v) {
    return __builtin_bit_cast(h16x2, __builtin_amdgcn_perm(0x64646464u, v, 0x07030602u));
}

DEV float sigmoidf_(float x) { return 1.f / (1.f + __expf(-x)); }
