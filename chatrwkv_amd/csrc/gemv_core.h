// Streaming GEMV building blocks for gfx950.
//
// Weight matrices are read in the input-contiguous layout: output row m is N consecutive
// elements (uint8 or fp16).  One wave owns a few output rows; lane l reads the 16-byte
// segments l, l+64, ... of each row (a wave reads 1 KiB contiguous per row per step), multiplies
// with the activation vector held in LDS and reduces across the wave with shuffles.  Nothing
// is shared between waves, so there are no atomics and results are deterministic.
//
// uint8 path: y[m] = rx[m] * sum_j xs[j] * (w[m][j] + 0.5) + mx[m] * S0 + S2 with
//   xs[j] = fp16(x[j] * ry[j]),  S0 = sum x[j],  S2 = sum x[j] * my[j].
// Bytes are widened two at a time to the fp16 values (1024 + b) with one v_perm_b32 and fed to
// v_dot2_f32_f16 (fp32 accumulate); the 1024 offset is removed afterwards with S1 = sum xs[j]:
//   sum xs[j] * (w + 0.5) = dot - 1023.5 * S1.
// (Turning the pairs into (b + 0.5) with a packed fp16 subtraction, which is exact and saves the third sum
// of every prologue, costs one more vector instruction per two weights in the streaming loop and was
// measured 2.7 % slower per token.)
#pragma once
#include "common.h"

// LDS layout of an activation vector of nseg = N/16 segments: the first 8 values of every
// segment are stored as 16-byte items [0, nseg), the last 8 as items [nseg, 2*nseg), so that
// the two ds_read_b128 of consecutive lanes hit consecutive 16-byte slots (conflict free).
DEV int xs_slot(int j, int nseg) {
    const int s = j >> 4, p = j & 15;
    return ((p >> 3) * nseg + s) * 8 + (p & 7);
}

struct VecSums {
    float s0, s1, s2;
};

// dot of 16 uint8 weights (as 1024 + b) with 16 fp16 activations.
DEV float dot16_u8(u32x4 w, h16x8 x0, h16x8 x1, float acc) {
    acc = __builtin_amdgcn_fdot2(u8pair_lo_1024(w.x), __builtin_shufflevector(x0, x0, 0, 1), acc, false);
    acc = __builtin_amdgcn_fdot2(u8pair_hi_1024(w.x), __builtin_shufflevector(x0, x0, 2, 3), acc, false);
    acc = __builtin_amdgcn_fdot2(u8pair_lo_1024(w.y), __builtin_shufflevector(x0, x0, 4, 5), acc, false);
    acc = __builtin_amdgcn_fdot2(u8pair_hi_1024(w.y), __builtin_shufflevector(x0, x0, 6, 7), acc, false);
    acc = __builtin_amdgcn_fdot2(u8pair_lo_1024(w.z), __builtin_shufflevector(x1, x1, 0, 1), acc, false);
    acc = __builtin_amdgcn_fdot2(u8pair_hi_1024(w.z), __builtin_shufflevector(x1, x1, 2, 3), acc, false);
    acc = __builtin_amdgcn_fdot2(u8pair_lo_1024(w.w), __builtin_shufflevector(x1, x1, 4, 5), acc, false);
    acc = __builtin_amdgcn_fdot2(u8pair_hi_1024(w.w), __builtin_shufflevector(x1, x1, 6, 7), acc, false);
    return acc;
}

// dot of 8 fp16 weights with 8 fp16 activations.
DEV float dot8_f16(u32x4 w, h16x8 x, float acc) {
    const h16x8 wh = __builtin_bit_cast(h16x8, w);
    acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(wh, wh, 0, 1), __builtin_shufflevector(x, x, 0, 1), acc, false);
    acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(wh, wh, 2, 3), __builtin_shufflevector(x, x, 2, 3), acc, false);
    acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(wh, wh, 4, 5), __builtin_shufflevector(x, x, 4, 5), acc, false);
    acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(wh, wh, 6, 7), __builtin_shufflevector(x, x, 6, 7), acc, false);
    return acc;
}

// A register tile of weights: U 16-byte segments of R rows per lane.  Loading and consuming are
// separate steps so that a kernel can put the loads of its first tile in flight *before* it
// builds the activation vector (weights do not depend on activations).  A segment is 16 bytes
// of a row for both weight types (16 uint8 or 8 fp16 values); nseg = row bytes / 16.
template <bool U8, int R, int U>
struct RowTile {
    u32x4 w[U][R];

    // No load is predicated: a lane past the end of the row re-reads its last segment (consume() skips
    // it), and with real == false (wave-uniform; a batch past the end of the wave's work) all lanes read
    // the first segment of the row, one cache line, and the tile is never consumed.  A load under a
    // branch would make the compiler's static s_waitcnt counting assume that it may not have been
    // issued, and every wait on an earlier load would then drain this tile too.
    DEV void load(const uint8_t *const (&rows)[R], int seg0, int nseg, bool real = true) {
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int s = real ? min(seg0 + lane + 64 * u, nseg - 1) : 0;
#pragma unroll
            for (int r = 0; r < R; ++r) w[u][r] = __builtin_nontemporal_load((const u32x4 *)(rows[r] + 16 * (size_t)s));
        }
    }

    // acc[r] += <row r segments [seg0, seg0 + 64 U), xs[r]>; xs in the layout of the weight type
    // (uint8: split lo/hi items, fp16: linear).
    DEV void consume(const h16 *const (&xs)[R], int seg0, int nseg, float (&acc)[R]) const {
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int s = seg0 + lane + 64 * u;
            if (s < nseg) {
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const h16x8 *xv = (const h16x8 *)xs[r];
                    if (U8)
                        acc[r] = dot16_u8(w[u][r], xv[s], xv[nseg + s], acc[r]);
                    else
                        acc[r] = dot8_f16(w[u][r], xv[s], acc[r]);
                }
            }
        }
    }
};

// Final value of a uint8 row from its raw dot product.
DEV float mm8_finish(float dot, const VecSums &S, float rx, float mx) {
    return rx * (dot - 1023.5f * S.s1) + mx * S.s0 + S.s2;
}
