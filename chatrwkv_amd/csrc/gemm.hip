// Prefill contraction y[T, M] = xs[T, N] @ W on fp16 MFMA (v_mfma_f32_32x32x16_f16).
//
// W is read in the input-contiguous layout (row m = N consecutive uint8 or fp16).  For
// uint8 weights each 16-byte global load is widened in registers to the exact fp16 values
// (b + 0.5) -- v_perm_b32 builds 1024 + b, one packed fp16 add removes 1023.5 -- and stored to
// LDS, so the matrix cores see a plain fp16 x fp16 product with fp32 accumulation.  The
// activation operand is the caller's x pre-multiplied by ry (mm8_prepare below), and the
// rank-1 corrections enter in the epilogue:
//     y[t, m] = rx[m] * acc[t, m] + mx[m] * S0[t] + S2[t],   S0 = sum_j x[t, j],  S2 = sum_j x[t, j] my[j].
//
// Tiling: BT x BM outputs per workgroup of 64 WT WM threads (WT x WM waves, each owning a
// (BT/WT) x (BM/WM) block built from 32x32 MFMA tiles), K step 64, LDS double buffered; both LDS
// tiles are [row][64 halves] with the eight 16-byte chunks of a row XOR-swizzled by (row & 7) so
// that the ds_read_b128 of 32 consecutive rows spreads over all banks.  A wave block of
// 128 x 128 needs 8 fragment reads per 16 MFMAs, which keeps the LDS pipe at half its peak; the
// 64 x 64 block of the small-tile variant needs 4 reads per 4 MFMAs and is LDS-bound, so it is
// only used when a larger tile would leave most CUs idle.
// Workgroup ids are remapped so that the workgroups which share a weight tile (same m0,
// different t0) run on the same XCD and the tile is fetched into that XCD's L2 once.
#include <algorithm>
#include "kernels.h"
#include "../../include/rwkv_hip_bench.h"
#include <cstdlib>
#include <mutex>

// Set-up that must run once per device (function attributes belong to the current device's copy of a kernel).
struct PerDeviceOnce {
    bool done[64] = {};
    // the slot of the current device, or nullptr when the device cannot be read (the caller then repeats the set-up)
    bool *slot() {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
        return &done[dev];
    }
};

namespace {

constexpr int BK = 64;  // halves per LDS row

// LDS address (in halves) of 16-byte chunk `chunk` (0..7) of tile row `row`.  Rows are 128 bytes.
// The chunk index is XORed with a per-row key chosen so that a ds_read_b128 / ds_write_b128 is
// conflict free both if the LDS serves 8 lanes x 16 B per cycle from 32 banks (8 consecutive
// rows must hit 8 different chunk slots) and if it serves 16 lanes from 64 banks (the 8 even and
// the 8 odd rows of 16 consecutive rows must each hit 8 different slots).
DEV int swz(int row, int chunk) { return row * BK + ((chunk ^ ((row & 7) ^ ((row >> 3) & 1))) << 3); }

// Epilogue of one output element: rank-1 corrections of the uint8 format, activation / residual, store.
// explicit fused multiply-adds: every kernel that ends in this epilogue rounds the same way
DEV float epi_affine(float v, float rxm, float mxm, float s0, float s2) { return __builtin_fmaf(rxm, v, __builtin_fmaf(mxm, s0, s2)); }
// v: the contraction after epi_affine; res / gate: the residual and gate inputs where ep.act uses them
DEV float epi_act(float v, float res, float gate, const GemmEpi &ep) {
    float o = round_h(v);
    switch (ep.act) {
        case ACT_SIGMOID: o = sigmoidf_(o); break;
        case ACT_RELU_SQ: o = fmaxf(o, 0.f); o = o * o; break;
        case ACT_SILU: o = o * sigmoidf_(o); break;
        case ACT_TANH: o = tanhf(o); break;
        case ACT_RESIDUAL: o = res + o; break;
        case ACT_GATED_RESIDUAL:
            o = round_h(gate * o);
            o = res + o;
            break;
        default: break;
    }
    if (ep.out_scale != 1.f) o = round_h(o) * ep.out_scale;
    return o;
}
DEV void gemm_epilogue(float v, int t, int m, float rxm, float mxm, const GemmEpi &ep, void *Y, int64_t ldy) {
    if (ep.rx) v = epi_affine(v, rxm, mxm, ep.s0[t], ep.s2[t]);
    if (ep.raw_f32) {
        ((float *)Y)[(size_t)t * ldy + m] = v;
        return;
    }
    float res = 0.f, gate = 0.f;
    if (ep.act == ACT_RESIDUAL || ep.act == ACT_GATED_RESIDUAL) res = h2f(ep.res[(size_t)t * ep.ldres + m]);
    if (ep.act == ACT_GATED_RESIDUAL) gate = h2f(ep.gate[(size_t)t * ep.ldgate + m]);
    const float o = epi_act(v, res, gate, ep);
    if (ep.out_dtype == RWKV_DT_F32)
        ((float *)Y)[(size_t)t * ldy + m] = round_h(o);
    else
        ((rwkv_half *)Y)[(size_t)t * ldy + m] = f2h(o);
}

// Split-K second pass: sums the KS partial slabs [KS][T][M] in slab order (deterministic) and runs the epilogue.
// Four consecutive outputs per thread (M % 4 == 0).
__global__ __launch_bounds__(256) void splitk_epilogue_kernel(int T, int M, int KS, const float *__restrict__ part, void *Y,
                                                              int64_t ldy, GemmEpi ep) {
    const int64_t n4 = (int64_t)T * M / 4, n = (int64_t)T * M;
    const int m4 = M / 4;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (int64_t)gridDim.x * 256) {
        const int t = (int)(i / m4), m = (int)(i - (int64_t)t * m4) * 4;
        f32x4 v = *(const f32x4 *)(part + 4 * i);
        for (int k = 1; k < KS; ++k) v += *(const f32x4 *)(part + (size_t)k * n + 4 * i);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float rxm = 1.f, mxm = 0.f;
            if (ep.rx) { rxm = h2f(ep.rx[m + e]); mxm = h2f(ep.mx[m + e]); }
            gemm_epilogue(v[e], t, m + e, rxm, mxm, ep, Y, ldy);
        }
    }
}

// The same pass for the direct-to-LDS launches, whose operands are all laid out for 16-byte accesses (dma_ok):
// eight consecutive outputs per thread, all slab loads of a thread in flight together, 16-byte loads of the
// residual / gate rows and 16-byte stores.  Same slab order and the same arithmetic per element as above.
template <int KS>
DEV void splitk_rows8(int T, int M, int ks_rt, const float *__restrict__ part, void *Y, int64_t ldy, const GemmEpi &ep,
                      int64_t first, int64_t stride) {
    const int64_t n8 = (int64_t)T * M / 8, n = (int64_t)T * M;
    const int m8 = M / 8, ks = KS ? KS : ks_rt;
    for (int64_t i = first; i < n8; i += stride) {
        const int t = (int)(i / m8), col = (int)(i - (int64_t)t * m8) * 8;
        f32x4 lo = *(const f32x4 *)(part + 8 * i), hi = *(const f32x4 *)(part + 8 * i + 4);
        if constexpr (KS > 0) {
            f32x4 pl[KS], ph[KS];
#pragma unroll
            for (int k = 1; k < KS; ++k) {
                pl[k] = *(const f32x4 *)(part + (size_t)k * n + 8 * i);
                ph[k] = *(const f32x4 *)(part + (size_t)k * n + 8 * i + 4);
            }
#pragma unroll
            for (int k = 1; k < KS; ++k) { lo += pl[k]; hi += ph[k]; }
        } else {
            for (int k = 1; k < ks; ++k) {
                lo += *(const f32x4 *)(part + (size_t)k * n + 8 * i);
                hi += *(const f32x4 *)(part + (size_t)k * n + 8 * i + 4);
            }
        }
        float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        if (ep.rx) {
            const h16x8 rx8 = *(const h16x8 *)(ep.rx + col), mx8 = *(const h16x8 *)(ep.mx + col);
            const float s0t = ep.s0[t], s2t = ep.s2[t];
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = epi_affine(v[e], (float)rx8[e], (float)mx8[e], s0t, s2t);
        }
        if (ep.raw_f32) {
            float *yo = (float *)Y + (size_t)t * ldy + col;
            *(f32x4 *)yo = f32x4{v[0], v[1], v[2], v[3]};
            *(f32x4 *)(yo + 4) = f32x4{v[4], v[5], v[6], v[7]};
            continue;
        }
        h16x8 res8 = {}, gate8 = {};
        if (ep.act == ACT_RESIDUAL || ep.act == ACT_GATED_RESIDUAL) res8 = *(const h16x8 *)(ep.res + (size_t)t * ep.ldres + col);
        if (ep.act == ACT_GATED_RESIDUAL) gate8 = *(const h16x8 *)(ep.gate + (size_t)t * ep.ldgate + col);
        float o[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = epi_act(v[e], (float)res8[e], (float)gate8[e], ep);
        if (ep.out_dtype == RWKV_DT_F32) {
            float *yo = (float *)Y + (size_t)t * ldy + col;
            *(f32x4 *)yo = f32x4{round_h(o[0]), round_h(o[1]), round_h(o[2]), round_h(o[3])};
            *(f32x4 *)(yo + 4) = f32x4{round_h(o[4]), round_h(o[5]), round_h(o[6]), round_h(o[7])};
        } else {
            h16x8 y8;
#pragma unroll
            for (int e = 0; e < 8; ++e) y8[e] = (h16)o[e];
            *(h16x8 *)((rwkv_half *)Y + (size_t)t * ldy + col) = y8;
        }
    }
}

DEV void splitk_rows8_any(int T, int M, int KS, const float *__restrict__ part, void *Y, int64_t ldy, const GemmEpi &ep,
                          int64_t first, int64_t stride) {
    switch (KS) {
        case 2: splitk_rows8<2>(T, M, KS, part, Y, ldy, ep, first, stride); break;
        case 4: splitk_rows8<4>(T, M, KS, part, Y, ldy, ep, first, stride); break;
        case 8: splitk_rows8<8>(T, M, KS, part, Y, ldy, ep, first, stride); break;
        default: splitk_rows8<0>(T, M, KS, part, Y, ldy, ep, first, stride); break;
    }
}

__global__ __launch_bounds__(256) void splitk_epilogue8_kernel(int T, int M, int KS, const float *__restrict__ part, void *Y,
                                                               int64_t ldy, GemmEpi ep) {
    splitk_rows8_any(T, M, KS, part, Y, ldy, ep, (int64_t)blockIdx.x * 256 + threadIdx.x, (int64_t)gridDim.x * 256);
}

template <bool W_U8, int BT, int BM, int WT, int WM, int PF, bool SPLIT>
DEV void gemm_body(int T, int N, int M, const h16 *__restrict__ A, int64_t lda, const void *__restrict__ Wv, int64_t ldw,
                   void *__restrict__ Y, int64_t ldy, const GemmEpi &ep, int nk_split, float *__restrict__ part) {
    constexpr int NT = 64 * WT * WM;                 // threads per workgroup
    constexpr int RA = NT / 8, RB8 = NT / 4;         // tile rows one pass of 16-byte loads covers (fp16 / uint8 rows)
    static_assert(BT % (32 * WT) == 0 && BM % (32 * WM) == 0 && BT % RA == 0 && BM % RB8 == 0, "tile");
    constexpr int MI = BT / (32 * WT), NI = BM / (32 * WM);  // 32x32 blocks per wave in each direction
    extern __shared__ __align__(16) unsigned char smem[];
    h16 *lA[2], *lB[2];
    lA[0] = (h16 *)smem;
    lB[0] = lA[0] + BT * BK;
    lA[1] = lB[0] + BM * BK;
    lB[1] = lA[1] + BT * BK;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wr = wave / WM, wc = wave % WM;
    // workgroup -> tile: hardware deals consecutive workgroup ids round-robin to the 8 XCDs;
    // undo that so each XCD gets a contiguous range of tiles, which walk the T direction first.
    const int tiles_t = (T + BT - 1) / BT;
    int bid = blockIdx.x;
    if ((gridDim.x & 7) == 0) bid = (bid & 7) * (gridDim.x >> 3) + (bid >> 3);
    const int t0 = (bid % tiles_t) * BT, m0 = (bid / tiles_t) * BM;
    if (m0 >= M) return;   // grouped launches size the grid for their widest member

    constexpr int A_LD = BT / RA;                    // 16-byte loads per thread for the A tile
    constexpr int B_LD = W_U8 ? BM / RB8 : BM / RA;  // 16-byte loads per thread for the W tile
    // PF k-tiles are in flight in registers (global latency under load is several k-tile times);
    // the LDS holds the tile being multiplied and the next one.
    u32x4 ra[PF][A_LD], rb[PF][B_LD];

    // split-K: blockIdx.y owns k-tiles [kbase, kbase + nk) and writes raw partial sums to its slab
    const int kbase = SPLIT ? blockIdx.y * nk_split : 0;
    auto load_tiles = [&](u32x4 (&qa)[A_LD], u32x4 (&qb)[B_LD], int kt) {
        const int k0 = (kbase + kt) * BK;
#pragma unroll
        for (int i = 0; i < A_LD; ++i) {
            const int row = (tid >> 3) + RA * i, ch = tid & 7;
            const int t = min(t0 + row, T - 1);
            qa[i] = *(const u32x4 *)(A + (size_t)t * lda + k0 + ch * 8);
        }
        if (W_U8) {
#pragma unroll
            for (int i = 0; i < B_LD; ++i) {
                const int row = (tid >> 2) + RB8 * i, ch = tid & 3;
                const int m = min(m0 + row, M - 1);
                qb[i] = *(const u32x4 *)((const uint8_t *)Wv + (size_t)m * ldw + k0 + ch * 16);  // a 64-byte half line: the other half is the next k-tile, kept in L1
            }
        } else {
#pragma unroll
            for (int i = 0; i < B_LD; ++i) {
                const int row = (tid >> 3) + RA * i, ch = tid & 7;
                const int m = min(m0 + row, M - 1);
                qb[i] = *(const u32x4 *)((const h16 *)Wv + (size_t)m * ldw + k0 + ch * 8);
            }
        }
    };
    auto store_tiles = [&](const u32x4 (&qa)[A_LD], const u32x4 (&qb)[B_LD], int buf) {
#pragma unroll
        for (int i = 0; i < A_LD; ++i) {
            const int row = (tid >> 3) + RA * i, ch = tid & 7;
            *(u32x4 *)(lA[buf] + swz(row, ch)) = qa[i];
        }
        if (W_U8) {
            const h16x2 off = {(h16)1023.5f, (h16)1023.5f};
#pragma unroll
            for (int i = 0; i < B_LD; ++i) {
                const int row = (tid >> 2) + RB8 * i, ch = tid & 3;
                u32x4 lo, hi;
                const uint32_t d[4] = {qb[i].x, qb[i].y, qb[i].z, qb[i].w};
                uint32_t o[8];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    o[2 * e] = __builtin_bit_cast(uint32_t, u8pair_lo_1024(d[e]) - off);
                    o[2 * e + 1] = __builtin_bit_cast(uint32_t, u8pair_hi_1024(d[e]) - off);
                }
                lo.x = o[0]; lo.y = o[1]; lo.z = o[2]; lo.w = o[3];
                hi.x = o[4]; hi.y = o[5]; hi.z = o[6]; hi.w = o[7];
                // rows r and r+2 share the XOR key's low bit: alternate which half goes first so the
                // 16 lanes of one write touch 16 different slots
                const int odd = (row >> 1) & 1;
                *(u32x4 *)(lB[buf] + swz(row, 2 * ch + odd)) = odd ? hi : lo;
                *(u32x4 *)(lB[buf] + swz(row, 2 * ch + 1 - odd)) = odd ? lo : hi;
            }
        } else {
#pragma unroll
            for (int i = 0; i < B_LD; ++i) {
                const int row = (tid >> 3) + RA * i, ch = tid & 7;
                *(u32x4 *)(lB[buf] + swz(row, ch)) = qb[i];
            }
        }
    };

    f32x16 acc[MI][NI];
#pragma unroll
    for (int a = 0; a < MI; ++a)
#pragma unroll
        for (int b = 0; b < NI; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;

    const int nk = SPLIT ? nk_split : N / BK;
    auto compute = [&](int buf) {
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            h16x8 fa[MI], fb[NI];
            const int ch = 2 * ks + (lane >> 5);
#pragma unroll
            for (int a = 0; a < MI; ++a) {
                const int row = wr * (BT / WT) + a * 32 + (lane & 31);
                fa[a] = *(const h16x8 *)(lA[buf] + swz(row, ch));
            }
#pragma unroll
            for (int b = 0; b < NI; ++b) {
                const int row = wc * (BM / WM) + b * 32 + (lane & 31);
                fb[b] = *(const h16x8 *)(lB[buf] + swz(row, ch));
            }
#pragma unroll
            for (int a = 0; a < MI; ++a)
#pragma unroll
                for (int b = 0; b < NI; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[a], fb[b], acc[a][b], 0, 0, 0);
        }
    };
    // Tile kt lives in register slot kt % PF from PF iterations before it is multiplied until it is written
    // to LDS buffer kt & 1 at the end of iteration kt - 1.  Every global load is issued unconditionally (past
    // the end the last k-tile is read again and never used): the compiler places its waits from a static
    // count of the loads issued after the one it needs, and a load under a branch would make it assume the
    // fewest, i.e. drain the whole prefetch queue before every LDS store.
#pragma unroll
    for (int p = 0; p < PF; ++p) load_tiles(ra[p], rb[p], min(p, nk - 1));
    store_tiles(ra[0], rb[0], 0);
    __syncthreads();
    for (int kt0 = 0; kt0 < nk; kt0 += PF) {
#pragma unroll
        for (int p = 0; p < PF; ++p) {
            const int kt = kt0 + p;
            load_tiles(ra[p], rb[p], min(kt + PF, nk - 1));  // slot freed when tile kt went to LDS
            if (kt < nk) compute(kt & 1);
            if (kt + 1 < nk) store_tiles(ra[(p + 1) % PF], rb[(p + 1) % PF], (kt + 1) & 1);
            __syncthreads();
        }
    }

    // epilogue: lane holds column m = .. + (lane & 31) and rows 8*(e/4) + 4*(lane>>5) + e%4
    float *slab = SPLIT ? part + (size_t)blockIdx.y * T * M : nullptr;
#pragma clang loop unroll(full)
    for (int b = 0; b < NI; ++b) {
        const int m = m0 + wc * (BM / WM) + b * 32 + (lane & 31);
        const bool m_ok = m < M;
        float rxm = 1.f, mxm = 0.f;
        if (!SPLIT && ep.rx && m_ok) { rxm = h2f(ep.rx[m]); mxm = h2f(ep.mx[m]); }
#pragma clang loop unroll(full)
        for (int a = 0; a < MI; ++a) {
#pragma clang loop unroll(full)
            for (int e = 0; e < 16; ++e) {
                const int t = t0 + wr * (BT / WT) + a * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                if (m_ok && t < T) {
                    if (SPLIT) slab[(size_t)t * M + m] = acc[a][b][e];
                    else gemm_epilogue(acc[a][b][e], t, m, rxm, mxm, ep, Y, ldy);
                }
            }
        }
    }
}

template <bool W_U8, int BT, int BM, int WT, int WM, int PF, bool SPLIT>
__global__ __launch_bounds__(64 * WT * WM) void gemm_kernel(int T, int N, int M, const h16 *__restrict__ A, int64_t lda,
                                                   const void *__restrict__ Wv, int64_t ldw, void *__restrict__ Y,
                                                   int64_t ldy, GemmEpi ep, int nk_split, float *__restrict__ part) {
    gemm_body<W_U8, BT, BM, WT, WM, PF, SPLIT>(T, N, M, A, lda, Wv, ldw, Y, ldy, ep, nk_split, part);
}

// ---- uint8 weights, large products: operands go from global memory straight into LDS ------------------------
// 256 x 256 tile, 8 waves (2 x 4, each 128 x 64), three LDS stages of one 64-deep k-tile each.  The loads are
// global_load_lds_dwordx4: one wave instruction copies 64 x 16 B into 1 KB of LDS without passing through
// registers, so no wave spends issue slots on ds_write or on holding prefetched tiles.  The weight tile stays
// uint8 in LDS (half the bytes of fp16) and becomes fp16 in the B fragments on the way to the matrix cores.
// LDS layout of a stage: A tile [256 rows][8 chunks of 16 B], chunk c of row r at slot c ^ ((r >> 1) & 7);
// W tile [256 rows][4 chunks of 16 B], chunk c of row r at slot c ^ ((r >> 2) & 3): both make the fragment reads
// (32 rows x one chunk per half-wave) hit every bank once.  The swizzle is applied on the global side: the lane
// that fills slot p of row r loads chunk p ^ key(r).
// Schedule of one k-tile: fragments of step ks + 1 are read while step ks multiplies (registers double-buffered);
// after the third of four steps every wave waits for its own loads of the next tile and meets the others at the
// one barrier, then issues the loads of tile kt + 3 into the stage it has just finished and reads the first
// fragments of tile kt + 1 while the fourth step multiplies.  LDS reads are inline asm with hand-placed
// s_waitcnt: the compiler waits for lgkmcnt(0) wherever older and newer reads are both outstanding.
// fp16 weights (W_U8 = false): the weight tile is laid out like the A tile (32 KB), a stage is 64 KB and two fit, so
// one tile is in flight while one multiplies.
// Tile TM x TN is 256 x 256 (wave tile 128 x 64: the long, wide products) or 128 x 128 (wave tile 64 x 32, a stage of
// 24 KB: products with too few 256 x 256 tiles for the chip run at full depth with these instead of splitting K).
// NW (waves per workgroup: 8, or 4 with 64 x 64 wave tiles) and NSTG (stages, 0 = the default above) exist for
// tuning runs.  Measured on the 128 x 128 tile with uint8 weights: four waves of 64 x 64 (a third fewer fragment
// reads per MFMA) 45.0 against 41.7 us on [1024 x 4096] x [4096 x 4096] and equal on launches of several rounds;
// four and five stages (tiles three and four ahead) 42.6 against 42.8 us, and 4-6 % slower on launches of several
// rounds, where only one workgroup then fits a CU.  Neither fragment reads nor load latency bound that tile.
constexpr int DT = 256, DM = 256;
template <bool W_U8, int TM, int TN, int NW = 8, int NSTG = 0> struct DmaCfg {
    static constexpr int A = TM * BK * 2, W = W_U8 ? TN * BK : TN * BK * 2, STAGE = A + W;
    static constexpr int NST = NSTG ? NSTG : (W_U8 || TM < 256) ? 3 : 2;
    static constexpr int AL = A / 1024 / NW, WL = W / 1024 / NW, LOADS = AL + WL;   // 1 KB loads per wave and tile
    static constexpr int WR = 2, WC = NW / 2;                            // waves: 2 rows x 4 (or 2) columns
    static constexpr int MI = TM / (32 * WR), NI = TN / (32 * WC);       // 32 x 32 blocks per wave
    static constexpr int STG_STRIDE = TN + 8;   // epilogue staging: 128 rows of TN floats, padded (see the epilogue)
    static constexpr size_t BODY = (size_t)NST * STAGE > (size_t)128 * STG_STRIDE * 4 ? (size_t)NST * STAGE : (size_t)128 * STG_STRIDE * 4;
    static constexpr size_t LDS = BODY + (W_U8 ? 2 * TM * 4 : 0);   // past the stages: the tile rows' sums s0, s2 (GemmEpi::parts)
};
// s_waitcnt immediates: vmcnt(n) alone, vmcnt(n) with lgkmcnt(0), lgkmcnt(n) alone
constexpr int vm_only(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }
constexpr int vm_lgkm0(int n) { return 0x0070 | (n & 15) | ((n >> 4) << 14); }
constexpr int lgkm_only(int n) { return 0xC07F | (n << 8); }

template <bool W_U8, bool SPLIT, int TM, int TN, int NW = 8, int NSTG = 0>
DEV void gemm_dma_body(int T, int N, int M, const h16 *__restrict__ A, int64_t lda, const void *__restrict__ Wv, int64_t ldw,
                       void *__restrict__ Y, int64_t ldy, const GemmEpi &ep, int nk_split, float *__restrict__ part, int split) {
    using Cfg = DmaCfg<W_U8, TM, TN, NW, NSTG>;
    constexpr int D_A = Cfg::A, D_STAGE = Cfg::STAGE, D_NST = Cfg::NST, AL = Cfg::AL, WL = Cfg::WL, MI = Cfg::MI, NI = Cfg::NI;
    static_assert((TM == 256 || TM == 128) && (TN == 256 || TN == 128), "tile");
    static_assert((NW == 8 || NW == 4) && 2 * TM <= 64 * NW && MI >= 2 && MI <= 4 && NI >= 1 && NI <= 2, "waves");
    extern __shared__ __align__(1024) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave / Cfg::WC, wc = wave % Cfg::WC;
    const int tiles_t = (T + TM - 1) / TM;
    int bid = blockIdx.x;
    if ((gridDim.x & 7) == 0) bid = (bid & 7) * (gridDim.x >> 3) + (bid >> 3);
    const int t0 = (bid % tiles_t) * TM, m0 = (bid / tiles_t) * TN;
    if (m0 >= M) return;   // grouped launches size the grid for their widest member
    const int kbase = SPLIT ? split * nk_split : 0, nk = SPLIT ? nk_split : N / BK;

    // load sources; rows past the end re-read the last row (never stored)
    const h16 *ga[AL];
#pragma unroll
    for (int i = 0; i < AL; ++i) {
        const int r = (wave * AL + i) * 8 + (lane >> 3), c = (lane & 7) ^ ((r >> 1) & 7);
        ga[i] = A + (size_t)min(t0 + r, T - 1) * lda + (size_t)kbase * BK + c * 8;
    }
    const unsigned char *gw[WL];   // byte pointers
#pragma unroll
    for (int i = 0; i < WL; ++i) {
        if (W_U8) {
            const int r = (wave * WL + i) * 16 + (lane >> 2), c = (lane & 3) ^ ((r >> 2) & 3);
            gw[i] = (const unsigned char *)Wv + (size_t)min(m0 + r, M - 1) * ldw + (size_t)kbase * BK + c * 16;
        } else {
            const int r = (wave * WL + i) * 8 + (lane >> 3), c = (lane & 7) ^ ((r >> 1) & 7);
            gw[i] = (const unsigned char *)((const h16 *)Wv + (size_t)min(m0 + r, M - 1) * ldw + (size_t)kbase * BK + c * 8);
        }
    }
    typedef __attribute__((address_space(1))) const void *gptr;
    typedef __attribute__((address_space(3))) void *lptr;
    // part 0 / 1: the halves of this wave's A loads, part 2: its weight loads; -1: all of them
    auto issue = [&](int kt, int so, int part) {
        unsigned char *base = smem + so;
#pragma unroll
        for (int i = 0; i < AL; ++i)
            if (part < 0 || part == (i >= (AL + 1) / 2 ? 1 : 0))
                __builtin_amdgcn_global_load_lds((gptr)(ga[i] + kt * BK), (lptr)(base + (wave * AL + i) * 1024), 16, 0, 0);
        if (part < 0 || part == 2) {
#pragma unroll
            for (int i = 0; i < WL; ++i)
                __builtin_amdgcn_global_load_lds((gptr)(gw[i] + kt * BK * (W_U8 ? 1 : 2)), (lptr)(base + D_A + (wave * WL + i) * 1024), 16, 0, 0);
        }
    };

    f32x16 acc[MI][NI];
#pragma unroll
    for (int a = 0; a < MI; ++a)
#pragma unroll
        for (int b = 0; b < NI; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;

    // fragment addresses within a stage; the swizzle keys depend on the lane only
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    uint32_t vA[4], vB[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        vA[ks] = lds0 + (wr * 32 * MI + (lane & 31)) * 128 + (((2 * ks + (lane >> 5)) ^ ((lane >> 1) & 7)) << 4);
        if (W_U8) vB[ks] = lds0 + D_A + (wc * 32 * NI + (lane & 31)) * 64 + ((ks ^ ((lane >> 2) & 3)) << 4) + (lane >> 5) * 8;
        else vB[ks] = lds0 + D_A + (wc * 32 * NI + (lane & 31)) * 128 + (((2 * ks + (lane >> 5)) ^ ((lane >> 1) & 7)) << 4);
    }
    h16x8 fa[2][MI], fbh[2][NI];   // fbh: B fragments of fp16 weights
    u32x2 rawb[2][NI];             // B fragments of uint8 weights, before conversion
    auto ldfrag = [&](int buf, int so, int ks) {
        const uint32_t pa = vA[ks] + so, pb = vB[ks] + so;
        if constexpr (W_U8) {
            asm volatile("ds_read_b64 %0, %1" : "=v"(rawb[buf][0]) : "v"(pb));
            if constexpr (NI > 1) asm volatile("ds_read_b64 %0, %1 offset:2048" : "=v"(rawb[buf][NI > 1 ? 1 : 0]) : "v"(pb));
        } else {
            asm volatile("ds_read_b128 %0, %1" : "=v"(fbh[buf][0]) : "v"(pb));
            if constexpr (NI > 1) asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(fbh[buf][NI > 1 ? 1 : 0]) : "v"(pb));
        }
        asm volatile("ds_read_b128 %0, %1" : "=v"(fa[buf][0]) : "v"(pa));
        asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(fa[buf][1]) : "v"(pa));
        if constexpr (MI > 2) {
            asm volatile("ds_read_b128 %0, %1 offset:8192" : "=v"(fa[buf][MI > 2 ? 2 : 0]) : "v"(pa));
            asm volatile("ds_read_b128 %0, %1 offset:12288" : "=v"(fa[buf][MI > 2 ? 3 : 0]) : "v"(pa));
        }
    };
    const h16x2 off = {(h16)1023.5f, (h16)1023.5f};
    // waits until only the newest fragment set (MI + NI reads) of this wave is outstanding: the one before has returned
    auto older_reads_done = [&]() {
        __builtin_amdgcn_s_waitcnt(lgkm_only(MI + NI));
        __builtin_amdgcn_sched_barrier(0);
    };
    auto multiply = [&](int cur) {
        h16x8 fb[NI];
#pragma unroll
        for (int b = 0; b < NI; ++b) {
            if constexpr (W_U8) {
                const u32x2 raw = rawb[cur][b];
                const h16x2 q0 = u8pair_lo_1024(raw.x) - off, q1 = u8pair_hi_1024(raw.x) - off;
                const h16x2 q2 = u8pair_lo_1024(raw.y) - off, q3 = u8pair_hi_1024(raw.y) - off;
                fb[b] = h16x8{q0.x, q0.y, q1.x, q1.y, q2.x, q2.y, q3.x, q3.y};
            } else {
                fb[b] = fbh[cur][b];
            }
        }
#pragma unroll
        for (int a = 0; a < MI; ++a)
#pragma unroll
            for (int b = 0; b < NI; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[cur][a], fb[b], acc[a][b], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    };

    // Every wave issues exactly LOADS loads per tile, so "vmcnt(LOADS n)" means "all but my newest n tiles have
    // landed".  Past the last tile the loads repeat it into a stage nobody reads any more, which keeps the counts static.
    // Three stages: while tile kt multiplies, tile kt + 1 has landed or is landing and the loads of tile kt + 2 are
    // issued in three parts between the MFMA steps, into the stage tile kt - 1 was read from (a burst of all of
    // them right after the barrier measured 2 % slower).  Two stages: tile kt + 2 can only go where tile kt is, so
    // its loads follow the barrier in one go.
    constexpr bool SPREAD = D_NST >= 3;
    constexpr int PD = SPREAD ? D_NST - 1 : 2;   // tiles in flight ahead of the one being multiplied
    issue(0, 0, -1);
    issue(min(1, nk - 1), D_STAGE, -1);
#pragma unroll
    for (int p = 2; p < PD; ++p) issue(min(p, nk - 1), p * D_STAGE, -1);
    // The input's row sums arrive as partial sums per column tile of the launch that produced it: this tile's rows
    // are added up here, in index order, while the first two tiles are in flight (the waits for these loads cover the
    // older tile loads too, so the counted waits below still hold).  Full depth: into LDS for the epilogue;
    // K split: the first column tile's first split writes the totals out for the second pass.
    bool lds_sums = false;
    if constexpr (W_U8) {
        if (ep.parts > 1 && (!SPLIT || (m0 == 0 && split == 0))) {
            lds_sums = !SPLIT;
            if (tid < 2 * TM) {
                const int row = tid & (TM - 1), which = tid / TM, t = min(t0 + row, T - 1);
                const float *p = (which ? ep.p2 : ep.p0) + (size_t)t * ep.parts;
                float tot = 0.f;
                for (int j = 0; j < ep.parts; j += 64) {   // parts % 4 == 0; up to 64 partial sums in flight per thread
                    f32x4 q[16];
#pragma unroll
                    for (int u = 0; u < 16; ++u) q[u] = j + 4 * u < ep.parts ? *(const f32x4 *)(p + j + 4 * u) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int u = 0; u < 16; ++u) tot = (((tot + q[u][0]) + q[u][1]) + q[u][2]) + q[u][3];
                }
                if constexpr (SPLIT) {
                    if (t0 + row < T) (which ? (float *)ep.s2 : (float *)ep.s0)[t] = tot;
                } else {
                    ((float *)(smem + Cfg::BODY))[tid] = tot;
                }
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(vm_only((PD - 1) * Cfg::LOADS));   // tile 0 has landed
    __builtin_amdgcn_s_barrier();
    int so = 0, sp = (D_NST - 1) * D_STAGE;   // the stage being read and (three stages and more) the one read before it
    // Second schedule (uint8 weights, and the large tile with fp16 weights; measured: [1024 x 4096] x [4096 x 4096]
    // uint8 57 -> 50 us, the large tile 1-4 % faster, the small tile with fp16 weights 10-15 % slower):
    // fragments are read TWO steps ahead of their MFMAs and the uint8 -> fp16 widening of step s + 1 is issued
    // right after the MFMAs of step s, so it runs while the matrix core works instead of between a fragment's
    // arrival and its MFMAs.  Step s uses register set s & 1 and refills it with step s + 2 once its MFMAs are
    // issued; all reads of a tile are therefore issued by its second step, where the one barrier per tile sits:
    // past it tile kt + 1 has landed for every wave and nobody reads tile kt's stage any more.
    constexpr bool AHEAD = W_U8 || TM == 256;
    if constexpr (AHEAD) {
        h16x8 fbc[2][NI];              // widened B fragments
        auto widen = [&](int buf) {
#pragma unroll
            for (int b = 0; b < NI; ++b) {
                if constexpr (W_U8) {
                    const u32x2 raw = rawb[buf][b];
                    const h16x2 q0 = u8pair_lo_1024(raw.x) - off, q1 = u8pair_hi_1024(raw.x) - off;
                    const h16x2 q2 = u8pair_lo_1024(raw.y) - off, q3 = u8pair_hi_1024(raw.y) - off;
                    fbc[buf][b] = h16x8{q0.x, q0.y, q1.x, q1.y, q2.x, q2.y, q3.x, q3.y};
                } else {
                    fbc[buf][b] = fbh[buf][b];
                }
            }
        };
        auto mfmas = [&](int buf) {
#pragma unroll
            for (int a = 0; a < MI; ++a)
#pragma unroll
                for (int b = 0; b < NI; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[buf][a], fbc[buf][b], acc[a][b], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        };
        auto reads_done = [&]() {
            __builtin_amdgcn_s_waitcnt(lgkm_only(0));
            __builtin_amdgcn_sched_barrier(0);
        };
        ldfrag(0, 0, 0);
        ldfrag(1, 0, 1);
        older_reads_done();
        widen(0);
        for (int kt = 0; kt < nk; ++kt) {
            const int sn = so + D_STAGE >= D_NST * D_STAGE ? 0 : so + D_STAGE;
            const int kl = min(kt + PD, nk - 1);
            // step 0
            mfmas(0);
            reads_done();
            widen(1);
            ldfrag(0, so, 2);
            if (SPREAD) issue(kl, sp, 0);
            __builtin_amdgcn_sched_barrier(0);
            // step 1
            mfmas(1);
            reads_done();
            widen(0);
            ldfrag(1, so, 3);
            if (SPREAD) issue(kl, sp, 1);
            __builtin_amdgcn_sched_barrier(0);
            // my part of tile kt + 1 has landed (newer: the A loads of tile kt + 2) and all my reads of tile kt are back
            __builtin_amdgcn_s_waitcnt(vm_lgkm0(SPREAD ? (PD - 2) * Cfg::LOADS + AL : 0));
            __builtin_amdgcn_s_barrier();
            if (!SPREAD) issue(kl, so, -1);
            // step 2
            mfmas(0);
            widen(1);
            ldfrag(0, sn, 0);
            if (SPREAD) issue(kl, sp, 2);
            __builtin_amdgcn_sched_barrier(0);
            // step 3
            mfmas(1);
            reads_done();
            widen(0);
            ldfrag(1, sn, 1);
            __builtin_amdgcn_sched_barrier(0);
            sp = so;
            so = sn;
        }
    } else {
        ldfrag(0, 0, 0);
        for (int kt = 0; kt < nk; ++kt) {
            const int sn = so + D_STAGE >= D_NST * D_STAGE ? 0 : so + D_STAGE;
            const int kl = min(kt + PD, nk - 1);
            ldfrag(1, so, 1);
            if (SPREAD) issue(kl, sp, 0);
            __builtin_amdgcn_sched_barrier(0);
            older_reads_done();
            multiply(0);
            ldfrag(0, so, 2);
            if (SPREAD) issue(kl, sp, 1);
            __builtin_amdgcn_sched_barrier(0);
            older_reads_done();
            multiply(1);
            ldfrag(1, so, 3);
            if (SPREAD) issue(kl, sp, 2);
            __builtin_amdgcn_sched_barrier(0);
            older_reads_done();
            multiply(0);
            // all my reads of this stage have returned and my part of tile kt + 1 has landed (with three stages tile
            // kt + 2 is in flight)
            __builtin_amdgcn_s_waitcnt(vm_lgkm0(SPREAD ? (PD - 1) * Cfg::LOADS : 0));
            __builtin_amdgcn_s_barrier();
            if (!SPREAD) issue(kl, so, -1);
            ldfrag(0, sn, 0);
            __builtin_amdgcn_sched_barrier(0);
            multiply(1);
            sp = so;
            so = sn;
        }
    }
    // vmcnt(0) lgkmcnt(0): nothing may land in LDS after the workgroup has gone -- and nothing in registers: the last
    // iteration has read a fragment set that nobody multiplies.  The compiler does not know that an inline-asm
    // ds_read writes its output later: to it those registers are dead from here on, and it reused them for the
    // epilogue's column index and addresses ahead of this wait (a read that returned late then overwrote the
    // index: an access far outside the buffers).  So the wait comes first, fenced against the scheduler, and every
    // fragment register stays "in use" until it has passed.
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x0070);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int buf = 0; buf < 2; ++buf) {
#pragma unroll
        for (int a = 0; a < MI; ++a) asm volatile("" ::"v"(fa[buf][a]));
#pragma unroll
        for (int b = 0; b < NI; ++b) {
            if constexpr (W_U8) asm volatile("" ::"v"(rawb[buf][b]));
            else asm volatile("" ::"v"(fbh[buf][b]));
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    // Each thread finishes eight consecutive outputs of one row: 16-byte loads of the residual / gate rows, 16-byte
    // stores, and a body small enough to stay in the instruction cache (per-element code for 128 accumulators
    // does not).
    constexpr int CPR = TN / 8, RPI = 64 * NW / CPR;   // 8-wide chunks per tile row; rows one pass of the workgroup covers
    const int cq = tid % CPR, col = m0 + cq * 8;
    const bool col_ok = col < M;   // M % 8 == 0
    h16x8 rx8, mx8, ery8 = {}, emy8 = {};
    if (W_U8 && col_ok) { rx8 = *(const h16x8 *)(ep.rx + col); mx8 = *(const h16x8 *)(ep.mx + col); }
    const bool emit = ep.emit_ry != nullptr;
    if (emit && col_ok) { ery8 = *(const h16x8 *)(ep.emit_ry + col); emy8 = *(const h16x8 *)(ep.emit_my + col); }
    const float *lsum = (const float *)(smem + Cfg::BODY);
    // trow: the row within the tile; a0 / a2: this thread's share of the emitted row sums
    auto finish8 = [&](int t, int trow, float (&v)[8], float &a0, float &a2) {
        if constexpr (W_U8) {
            const float s0t = lds_sums ? lsum[trow] : ep.s0[t], s2t = lds_sums ? lsum[TM + trow] : ep.s2[t];
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = epi_affine(v[e], (float)rx8[e], (float)mx8[e], s0t, s2t);
        }
        if (ep.raw_f32) {
            float *yo = (float *)Y + (size_t)t * ldy + col;
            *(f32x4 *)yo = f32x4{v[0], v[1], v[2], v[3]};
            *(f32x4 *)(yo + 4) = f32x4{v[4], v[5], v[6], v[7]};
            return;
        }
        h16x8 res8 = {}, gate8 = {};
        if (ep.act == ACT_RESIDUAL || ep.act == ACT_GATED_RESIDUAL) res8 = *(const h16x8 *)(ep.res + (size_t)t * ep.ldres + col);
        if (ep.act == ACT_GATED_RESIDUAL) gate8 = *(const h16x8 *)(ep.gate + (size_t)t * ep.ldgate + col);
        float o[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = epi_act(v[e], (float)res8[e], (float)gate8[e], ep);
        if (emit) {
            // what the scaling pass of the next product would make of the fp16 output: fp16(y * ry), sum y, sum y * my
            h16x8 y8;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float yf = (float)(h16)o[e];
                y8[e] = (h16)(yf * (float)ery8[e]);
                a0 += yf;
                a2 += yf * (float)emy8[e];
            }
            *(h16x8 *)((rwkv_half *)Y + (size_t)t * ldy + col) = y8;
        } else if (ep.out_dtype == RWKV_DT_F32) {
            float *yo = (float *)Y + (size_t)t * ldy + col;
            *(f32x4 *)yo = f32x4{round_h(o[0]), round_h(o[1]), round_h(o[2]), round_h(o[3])};
            *(f32x4 *)(yo + 4) = f32x4{round_h(o[4]), round_h(o[5]), round_h(o[6]), round_h(o[7])};
        } else {
            h16x8 y8;
#pragma unroll
            for (int e = 0; e < 8; ++e) y8[e] = (h16)o[e];
            *(h16x8 *)((rwkv_half *)Y + (size_t)t * ldy + col) = y8;
        }
    };

    if constexpr (SPLIT) {
        // partial sums go to this split's fp32 slab; splitk_epilogue8_kernel adds the slabs and finishes
        float *slab = part + (size_t)split * T * M;
#pragma unroll
        for (int b = 0; b < NI; ++b) {
            const int m = m0 + wc * 32 * NI + b * 32 + (lane & 31);
#pragma unroll
            for (int a = 0; a < MI; ++a)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int t = t0 + wr * 32 * MI + a * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                    if (m < M && t < T) slab[(size_t)t * M + m] = acc[a][b][e];
                }
        }
    } else {
        // The accumulators pass through LDS (free now), 128 tile rows at a time.
        constexpr int SW = Cfg::STG_STRIDE;   // row stride in floats: 4 rows apart = 32 banks apart for the two half-waves
        constexpr int WROWS = 32 * MI;        // tile rows of one wave row
        float *stg = (float *)smem;
        __syncthreads();   // every wave has read its last fragments
#pragma unroll 1
        for (int h = 0; h < TM / 128; ++h) {
            if ((wr * WROWS) / 128 == h) {
#pragma unroll
                for (int b = 0; b < NI; ++b)
#pragma unroll
                    for (int a = 0; a < MI; ++a)
#pragma unroll
                        for (int e = 0; e < 16; ++e)
                            stg[(wr * WROWS - h * 128 + a * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3)) * SW + wc * 32 * NI + b * 32 + (lane & 31)] =
                                acc[a][b][e];
            }
            __syncthreads();
#pragma unroll 1
            for (int it = 0; it < 128 / RPI; ++it) {
                const int row = it * RPI + tid / CPR, t = t0 + h * 128 + row;
                const bool valid = t < T && col_ok;
                float a0 = 0.f, a2 = 0.f;
                if (valid) {
                    const f32x4 v0 = *(const f32x4 *)(stg + row * SW + cq * 8), v1 = *(const f32x4 *)(stg + row * SW + cq * 8 + 4);
                    float v[8] = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
                    finish8(t, h * 128 + row, v, a0, a2);
                }
                if (emit) {   // the CPR threads of a row are neighbours in one wave; every lane takes part
                    a0 = row16_sum(a0);
                    a2 = row16_sum(a2);
                    if constexpr (CPR == 32) { a0 += __shfl_xor(a0, 16, WAVE); a2 += __shfl_xor(a2, 16, WAVE); }
                    if (valid && cq == 0) {
                        const size_t pi = (size_t)t * ((M + TN - 1) / TN) + m0 / TN;
                        ep.emit_s0[pi] = a0;
                        ep.emit_s2[pi] = a2;
                    }
                }
            }
            __syncthreads();
        }
    }
}

template <bool W_U8, bool SPLIT, int TM, int TN, int NW, int NSTG>
__global__ __launch_bounds__(64 * NW) void gemm_dma_kernel(int T, int N, int M, const h16 *__restrict__ A, int64_t lda,
                                                           const void *__restrict__ W, int64_t ldw, void *__restrict__ Y,
                                                           int64_t ldy, GemmEpi ep, int nk_split, float *__restrict__ part) {
    gemm_dma_body<W_U8, SPLIT, TM, TN, NW, NSTG>(T, N, M, A, lda, W, ldw, Y, ldy, ep, nk_split, part, SPLIT ? blockIdx.y : 0);
}

// Up to four contractions [T, N] x [N, M_i] in one launch (blockIdx.y picks the operands), at full depth: short
// calls, where each of them alone would split K and need a reduction pass.
struct GemmGroup {
    const h16 *A[4];
    const void *W[4];
    void *Y[4];
    int64_t lda, ldw[4];
    int M[4];
    float *part[4];   // split-K slabs of member i, [splits][T][M_i] (direct-to-LDS group only)
    int nk_split;
    GemmEpi ep[4];
};

template <bool W_U8, int BT, int BM, int WT, int WM, int PF>
__global__ __launch_bounds__(64 * WT * WM) void gemm_group_kernel(int T, int N, GemmGroup g) {
    const int gi = blockIdx.y, M = g.M[gi];
    gemm_body<W_U8, BT, BM, WT, WM, PF, false>(T, N, M, g.A[gi], g.lda, g.W[gi], g.ldw[gi], g.Y[gi], M, g.ep[gi], N / BK,
                                               nullptr);
}

// the same through the direct-to-LDS kernel; blockIdx.z is the k split when the group has too few tiles for the chip
template <bool W_U8, bool SPLIT, int TM, int TN>
__global__ __launch_bounds__(512) void gemm_dma_group_kernel(int T, int N, GemmGroup g) {
    const int gi = blockIdx.y, M = g.M[gi];
    gemm_dma_body<W_U8, SPLIT, TM, TN>(T, N, M, g.A[gi], g.lda, g.W[gi], g.ldw[gi], g.Y[gi], M, g.ep[gi], SPLIT ? g.nk_split : N / BK,
                                       g.part[gi], SPLIT ? blockIdx.z : 0);
}

template <bool W_U8, int TM, int TN>
int launch_dma_group(const GemmGroup &g, int n, int64_t T, int64_t N, int64_t grid_x, int ks, hipStream_t st) {
    constexpr size_t lds = DmaCfg<W_U8, TM, TN>::LDS;
    static PerDeviceOnce once;
    bool *attr_done = once.slot();
    if (!attr_done || !*attr_done) {
        hipError_t e = hipFuncSetAttribute((const void *)gemm_dma_group_kernel<W_U8, false, TM, TN>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e == hipSuccess)
            e = hipFuncSetAttribute((const void *)gemm_dma_group_kernel<W_U8, true, TM, TN>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)lds);
        if (e != hipSuccess) return (int)e;
        if (attr_done) *attr_done = true;
    }
    const dim3 grid((unsigned)grid_x, (unsigned)n, (unsigned)ks);
    if (ks > 1) hipLaunchKernelGGL((gemm_dma_group_kernel<W_U8, true, TM, TN>), grid, dim3(512), lds, st, (int)T, (int)N, g);
    else hipLaunchKernelGGL((gemm_dma_group_kernel<W_U8, false, TM, TN>), grid, dim3(512), lds, st, (int)T, (int)N, g);
    return RWKV_OK;
}

// second pass of a split group launch: member blockIdx.y, as splitk_epilogue8_kernel
__global__ __launch_bounds__(256) void splitk_group_epilogue8_kernel(int T, int KS, GemmGroup g) {
    const int gi = blockIdx.y;
    splitk_rows8_any(T, g.M[gi], KS, g.part[gi], g.Y[gi], g.M[gi], g.ep[gi], (int64_t)blockIdx.x * 256 + threadIdx.x,
                     (int64_t)gridDim.x * 256);
}

struct PrepGroup {
    const rwkv_half *x[4], *ry[4], *my[4];
    rwkv_half *xs[4];
    float *s0[4], *s2[4];
};

// xs[t, j] = fp16(x[t, j] * ry[j]);  s0[t] = sum_j x[t, j];  s2[t] = sum_j x[t, j] * my[j].  One workgroup (four
// waves) per row: a 16384-wide row per wave left the memory system with four waves per CU to draw from.
__global__ __launch_bounds__(256) void mm8_prepare_kernel(int T, int N, const rwkv_half *__restrict__ x, int64_t ldx,
                                                          const rwkv_half *__restrict__ ry,
                                                          const rwkv_half *__restrict__ my, rwkv_half *__restrict__ xs,
                                                          float *__restrict__ s0, float *__restrict__ s2) {
    __shared__ float red[8];
    const int t = blockIdx.x, lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    float a0 = 0.f, a2 = 0.f;
    for (int j = threadIdx.x * 8; j < N; j += 256 * 8) {
        const u32x4 xv = *(const u32x4 *)(x + (size_t)t * ldx + j);
        const u32x4 rv = *(const u32x4 *)(ry + j);
        const u32x4 mv = *(const u32x4 *)(my + j);
        const h16x8 xh = __builtin_bit_cast(h16x8, xv), rh = __builtin_bit_cast(h16x8, rv),
                    mh = __builtin_bit_cast(h16x8, mv);
        h16x8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float xf = (float)xh[e];
            o[e] = (h16)(xf * (float)rh[e]);
            a0 += xf;
            a2 += xf * (float)mh[e];
        }
        *(u32x4 *)(xs + (size_t)t * N + j) = __builtin_bit_cast(u32x4, o);
    }
    a0 = wave_sum(a0);
    a2 = wave_sum(a2);
    if (lane == 0) { red[wid] = a0; red[4 + wid] = a2; }
    __syncthreads();
    if (threadIdx.x == 0) {
        s0[t] = (red[0] + red[1]) + (red[2] + red[3]);
        s2[t] = (red[4] + red[5]) + (red[6] + red[7]);
    }
}

// the same for up to four (x, matrix) pairs in one launch: blockIdx.y picks the pair
__global__ __launch_bounds__(256) void mm8_prepare_group_kernel(int T, int N, PrepGroup g) {
    const int gi = blockIdx.y;
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (t >= T) return;
    const rwkv_half *x = g.x[gi], *ry = g.ry[gi], *my = g.my[gi];
    rwkv_half *xs = g.xs[gi];
    float a0 = 0.f, a2 = 0.f;
    for (int j = lane * 8; j < N; j += 64 * 8) {
        const h16x8 xh = *(const h16x8 *)(x + (size_t)t * N + j), rh = *(const h16x8 *)(ry + j), mh = *(const h16x8 *)(my + j);
        h16x8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float xf = (float)xh[e];
            o[e] = (h16)(xf * (float)rh[e]);
            a0 += xf;
            a2 += xf * (float)mh[e];
        }
        *(h16x8 *)(xs + (size_t)t * N + j) = o;
    }
    a0 = wave_sum(a0);
    a2 = wave_sum(a2);
    if (lane == 0) { g.s0[gi][t] = a0; g.s2[gi][t] = a2; }
}



// ---- calls of 2 .. 16 rows: every weight row streamed once ---------------------------------------------------
// A ragged last prompt chunk (rwkv/utils.py:98-101) or a short chat turn has a handful of tokens: with 128-row
// tiles the contraction kernels spend their time on empty rows and a call costs several one-token steps.  Here
// a workgroup of 16 waves takes 16 output rows at a time and splits K over its waves: wave w owns the k-chunks
// w, w + 16, ... (64 wide for uint8 rows, 32 for fp16 rows); per chunk a lane loads 16 bytes of one weight row
// (lane = row + 16 q: the four lanes of a row cover 64 contiguous bytes) and the matching 16 / 8 activation values
// of one token (lane = token + 16 q, rows past T repeat the last one), widens uint8 to the exact fp16 value b + 1/2
// and issues v_mfma_f32_16x16x32_f16 with the weights as the first and the activations as the second operand, so
// that lane (token j, q) ends with rows 4 q .. 4 q + 3 of token j.  The 16 partial 16 x 16 blocks are added in wave
// order through LDS (deterministic), and 256 threads run the same epilogue as the large kernels.  Activations come
// from L2 (T x N values, re-read per row group); weights from HBM, each byte once.
struct SkinnyGroup {
    const h16 *A[4];
    const void *W[4];
    void *Y[4];
    int64_t lda, ldw[4], ldy[4];
    int M[4];
    GemmEpi ep[4];
};

// NCI > 0: a wave owns at most NCI chunks and keeps their activation values in registers for all its row groups
// (rows of up to 16 * NCI chunks: the loop then issues weight loads only); NCI == 0: any row length, activations
// re-read from L2 for every row group.
template <bool W_U8, int NCI>
__global__ __launch_bounds__(1024) void skinny_kernel(int T, int N, SkinnyGroup g) {
    __shared__ float red[16][64][4];
    const int gi = blockIdx.y, M = g.M[gi];
    const h16 *__restrict__ A = g.A[gi];
    const unsigned char *__restrict__ W = (const unsigned char *)g.W[gi];
    const int64_t lda = g.lda, ldw = g.ldw[gi];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int sub = lane & 15, q = lane >> 4;
    constexpr int CK = W_U8 ? 64 : 32;               // k values per chunk
    const int nchunks = N / CK;
    const int ngroups = (M + 15) >> 4;
    const h16 *arow = A + (size_t)min(sub, T - 1) * lda;   // this lane's token
    const h16x2 off = {(h16)1023.5f, (h16)1023.5f};
    constexpr int NB = NCI > 0 ? NCI : 4;            // chunks loaded before any is multiplied
    auto load_x = [&](int c, h16x8 &x0, h16x8 &x1) {
        if (W_U8) {
            x0 = *(const h16x8 *)(arow + (size_t)c * 64 + 16 * q);
            x1 = *(const h16x8 *)(arow + (size_t)c * 64 + 16 * q + 8);
        } else {
            x0 = *(const h16x8 *)(arow + (size_t)c * 32 + 8 * q);
            x1 = x0;
        }
    };
    auto load_w = [&](const unsigned char *wrow, int c) {
        if (W_U8) return __builtin_nontemporal_load((const u32x4 *)(wrow + (size_t)c * 64 + 16 * q));
        return __builtin_nontemporal_load((const u32x4 *)(wrow + ((size_t)c * 32 + 8 * q) * 2));
    };
    auto multiply = [&](u32x4 wv, h16x8 x0, h16x8 x1, f32x4 &acc) {
        if (W_U8) {
            const h16x2 a0 = u8pair_lo_1024(wv.x) - off, a1 = u8pair_hi_1024(wv.x) - off;
            const h16x2 a2 = u8pair_lo_1024(wv.y) - off, a3 = u8pair_hi_1024(wv.y) - off;
            const h16x2 b0 = u8pair_lo_1024(wv.z) - off, b1 = u8pair_hi_1024(wv.z) - off;
            const h16x2 b2 = u8pair_lo_1024(wv.w) - off, b3 = u8pair_hi_1024(wv.w) - off;
            const h16x8 wa = {a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
            const h16x8 wb = {b0.x, b0.y, b1.x, b1.y, b2.x, b2.y, b3.x, b3.y};
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(wa, x0, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(wb, x1, acc, 0, 0, 0);
        } else {
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h16x8, wv), x0, acc, 0, 0, 0);
        }
    };
    // chunks past the end of the row repeat the last one and multiply zeros: no branch sits between the loads and
    // their use (loads would be sunk behind it, one chunk in flight at a time)
    h16x8 rx0[NB], rx1[NB];
    if (NCI > 0) {
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            load_x(min(wave + 16 * i, nchunks - 1), rx0[i], rx1[i]);
            if (wave + 16 * i >= nchunks) { rx0[i] = h16x8{}; rx1[i] = h16x8{}; }
        }
    }
    for (int grp = blockIdx.x; grp < ngroups; grp += gridDim.x) {
        const int m0 = grp << 4;
        const unsigned char *wrow = W + (size_t)min(m0 + sub, M - 1) * ldw * (W_U8 ? 1 : 2);
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        if (NCI > 0) {
            u32x4 wv[NB];
#pragma unroll
            for (int i = 0; i < NB; ++i) wv[i] = load_w(wrow, min(wave + 16 * i, nchunks - 1));
#pragma unroll
            for (int i = 0; i < NB; ++i) multiply(wv[i], rx0[i], rx1[i], acc);
        } else {
            for (int c0 = wave; c0 < nchunks; c0 += 16 * NB) {
                u32x4 wv[NB];
                h16x8 x0[NB], x1[NB];
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    const int c = min(c0 + 16 * i, nchunks - 1);
                    wv[i] = load_w(wrow, c);
                    load_x(c, x0[i], x1[i]);
                }
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    if (c0 + 16 * i >= nchunks) { x0[i] = h16x8{}; x1[i] = h16x8{}; }
                    multiply(wv[i], x0[i], x1[i], acc);
                }
            }
        }
        __syncthreads();                                          // the previous group's sums have been read
        *(f32x4 *)&red[wave][lane][0] = acc;
        __syncthreads();
        if (threadIdx.x < 256) {
            const int l = threadIdx.x & 63, r = threadIdx.x >> 6;
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < 16; ++w) v += red[w][l][r];
            const int m = m0 + 4 * (l >> 4) + r, t = l & 15;
            if (m < M && t < T) {
                const GemmEpi &ep = g.ep[gi];
                float rxm = 1.f, mxm = 0.f;
                if (ep.rx) { rxm = h2f(ep.rx[m]); mxm = h2f(ep.mx[m]); }
                gemm_epilogue(v, t, m, rxm, mxm, ep, g.Y[gi], g.ldy[gi]);
            }
        }
    }
}

constexpr int SKINNY_MAX_ROWS = 16;

// what skinny_kernel assumes of one product: whole chunks, 16-byte aligned rows for its 16-byte loads
bool skinny_ok(bool w_u8, int64_t T, int64_t N, const void *A, int64_t lda, const void *W, int64_t ldw, const GemmEpi &ep) {
    auto a16 = [](const void *p) { return (((uintptr_t)p) & 15) == 0; };
    if (T < 2 || T > SKINNY_MAX_ROWS || N < 64 || (N % 64)) return false;
    if ((lda & 7) || (ldw & (w_u8 ? 15 : 7)) || !a16(A) || !a16(W)) return false;
    if (w_u8 && (!ep.rx || !ep.mx || !ep.s0 || !ep.s2)) return false;
    if (!w_u8 && ep.rx) return false;
    const char *e = getenv("RWKV_NO_SKINNY");                     // tuning: send short calls through the tile kernels
    return !(e && *e == '1');
}

int skinny_launch(bool w_u8, int n, int64_t T, int64_t N, const SkinnyGroup &g, hipStream_t st) {
    int maxg = 1;
    for (int i = 0; i < n; ++i) maxg = std::max(maxg, (g.M[i] + 15) / 16);
    const dim3 grid((unsigned)std::min(maxg, 2 * num_cu()), (unsigned)n);
    const int64_t per_wave = (N / (w_u8 ? 64 : 32) + 15) / 16;    // chunks a wave owns
#define RWKV_SKINNY(NCI)                                                                                         \
    do {                                                                                                         \
        if (w_u8) hipLaunchKernelGGL((skinny_kernel<true, NCI>), grid, dim3(1024), 0, st, (int)T, (int)N, g);   \
        else hipLaunchKernelGGL((skinny_kernel<false, NCI>), grid, dim3(1024), 0, st, (int)T, (int)N, g);       \
    } while (0)
    if (per_wave <= 1) RWKV_SKINNY(1);
    else if (per_wave <= 2) RWKV_SKINNY(2);
    else if (per_wave <= 4) RWKV_SKINNY(4);
    else if (per_wave <= 8) RWKV_SKINNY(8);
    else RWKV_SKINNY(0);
#undef RWKV_SKINNY
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

// ---- narrow outputs: [T, N] x [N, M] with M of a LoRA rank and fp16 weights ------------------------------------
// The first stage of a low-rank product (RWKV-6 mixing and decay LoRA, RWKV-7's four) has thousands of input columns
// and a few dozen to a few hundred outputs: a handful of 128 x 128 tiles, which the tile kernels can only spread
// over the chip by splitting K and adding the slabs in a second launch.  Here a workgroup of eight waves takes a
// 16 x 16 block of the output and splits K over its waves: wave w owns the 32-wide k-chunks w, w + 8, ...; per
// chunk a lane loads 16 bytes of one weight row and of one activation row (lane = row + 16 q: the four lanes of a
// row cover 64 contiguous bytes), sixteen chunks in flight, and issues v_mfma_f32_16x16x32_f16 with the weights as
// the first operand, so that lane (token j, q) ends with outputs 4 q .. 4 q + 3 of token j.  The eight partial
// blocks are added in wave order through LDS (deterministic) and 64 threads round, apply the activation and store
// 8 bytes each.  Operands come from L2: the weights are read once per 16 rows of the call, the activation once per
// 16 outputs, so the kernel serves calls of up to NARROW_MAX_T rows ([256 x 4096] x [4096 x 160]: 9 us against
// 14 us for the K-split tiles and their second pass; at 1024 rows the tiles win, 23 against 14 us).
__global__ __launch_bounds__(512) void narrow_kernel(int T, int N, int M, const h16 *__restrict__ A, int64_t lda,
                                                     const h16 *__restrict__ W, int64_t ldw, rwkv_half *__restrict__ Y,
                                                     int64_t ldy, GemmEpi ep) {
    __shared__ f32x4 red[8][64];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int sub = lane & 15, q = lane >> 4;
    const int t0 = blockIdx.x * 16, m0 = blockIdx.y * 16;
    const h16 *arow = A + (size_t)min(t0 + sub, T - 1) * lda + 8 * q;
    const h16 *wrow = W + (size_t)min(m0 + sub, M - 1) * ldw + 8 * q;
    const int nchunks = N / 32;
    constexpr int NB = 16;   // chunks in flight per wave: a 4096-wide row is one round
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    // chunks past the end repeat the last one and multiply zeros (no branch between the loads and their use)
    for (int c0 = wave; c0 < nchunks; c0 += 8 * NB) {
        h16x8 wv[NB], xv[NB];
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const int c = min(c0 + 8 * i, nchunks - 1);
            wv[i] = *(const h16x8 *)(wrow + (size_t)c * 32);
            xv[i] = *(const h16x8 *)(arow + (size_t)c * 32);
        }
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            if (c0 + 8 * i >= nchunks) xv[i] = h16x8{};
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(wv[i], xv[i], acc, 0, 0, 0);
        }
    }
    red[wave][lane] = acc;
    __syncthreads();
    if (wave == 0) {
        f32x4 v = red[0][lane];
#pragma unroll
        for (int w = 1; w < 8; ++w) v += red[w][lane];
        const int t = t0 + sub, m = m0 + 4 * q;
        if (t < T && m < M) {   // M % 4 == 0
            h16x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (h16)epi_act(v[e], 0.f, 0.f, ep);
            *(h16x4 *)((h16 *)Y + (size_t)t * ldy + m) = o;
        }
    }
}

// narrow_kernel's operands: fp16 weights, at most NARROW_MAX_M outputs, rows of whole 32-wide chunks laid out for
// 16-byte loads, an epilogue without residual or gate, fp16 out.  RWKV_NO_NARROW=1 sends these through the tile
// kernels (tuning).
constexpr int NARROW_MAX_M = 192, NARROW_MAX_T = 512;
bool narrow_ok(bool w_u8, int64_t T, int64_t N, int64_t M, const void *A, int64_t lda, const void *W, int64_t ldw, const void *Y,
               int64_t ldy, const GemmEpi &ep) {
    auto a16 = [](const void *p) { return (((uintptr_t)p) & 15) == 0; };
    if (w_u8 || ep.rx || T <= SKINNY_MAX_ROWS || T > NARROW_MAX_T || M > NARROW_MAX_M || (M & 3) || N < 1024 || (N % 32)) return false;
    if ((lda & 7) || (ldw & 7) || (ldy & 3) || !a16(A) || !a16(W) || (((uintptr_t)Y) & 7)) return false;
    if (ep.act == ACT_RESIDUAL || ep.act == ACT_GATED_RESIDUAL || ep.raw_f32 || ep.out_dtype != RWKV_DT_F16) return false;
    const char *e = getenv("RWKV_NO_NARROW");
    return !(e && *e == '1');
}

}  // namespace

namespace {

template <bool W_U8, int BT, int BM, int WT, int WM, int PF>
int launch_cfg(int64_t T, int64_t N, int64_t M, const rwkv_half *A, int64_t lda, const void *W, int64_t ldw, void *Y,
               int64_t ldy, const GemmEpi &ep, hipStream_t st) {
    constexpr size_t lds = 2 * (size_t)(BT + BM) * BK * sizeof(h16);
    static PerDeviceOnce once;
    bool *attr_done = once.slot();
    if (lds > 64 * 1024 && (!attr_done || !*attr_done)) {
        hipError_t e = hipFuncSetAttribute((const void *)gemm_kernel<W_U8, BT, BM, WT, WM, PF, false>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        if (attr_done) *attr_done = true;
    }
    const int64_t tiles = ((T + BT - 1) / BT) * ((M + BM - 1) / BM);
    // Too few tiles to fill the chip (short prompts, narrow matrices): split the contraction over KS
    // workgroups per tile; partial sums go to fp32 slabs and a second pass reduces them in slab order.
    int ks = 1;
    const int nk = (int)(N / BK);
    // up to 128 tiles: split until every CU has a workgroup; up to 256 tiles (at most one workgroup per CU, which
    // leaves a CU's four waves waiting on their own loads): split in two, +12-18 % on 1024 x 4096 x 4096,
    // 1024 x 16384 x 4096 and 256 x 4096 x 16384
    const int want = tiles <= 128 ? 256 : 512;
    if (ep.splitk_ws && tiles <= 256 && lds <= 64 * 1024 && (M & 3) == 0) {
        // the smallest split that reaches that many workgroups (slab traffic grows with the split)
        for (int c = 2; c <= 8; c <<= 1) {
            if (nk % c || nk / c < 8) break;                                      // whole k-tiles, several per split
            if ((size_t)c * T * M * sizeof(float) > ep.splitk_bytes) break;       // slabs must fit
            ks = c;
            if (tiles * c >= want) break;
        }
    }
    if (ks > 1) {
        hipLaunchKernelGGL((gemm_kernel<W_U8, BT, BM, WT, WM, PF, true>), dim3((unsigned)tiles, (unsigned)ks), dim3(64 * WT * WM), lds, st,
                           (int)T, (int)N, (int)M, (const h16 *)A, lda, W, ldw, Y, ldy, ep, nk / ks, ep.splitk_ws);
        const int64_t n = T * M;
        const unsigned blocks = (unsigned)((n + 1023) / 1024 < 16384 ? (n + 1023) / 1024 : 16384);
        hipLaunchKernelGGL(splitk_epilogue_kernel, dim3(blocks), dim3(256), 0, st, (int)T, (int)M, ks, ep.splitk_ws, Y, ldy, ep);
    } else {
        hipLaunchKernelGGL((gemm_kernel<W_U8, BT, BM, WT, WM, PF, false>), dim3((unsigned)tiles), dim3(64 * WT * WM), lds, st, (int)T,
                           (int)N, (int)M, (const h16 *)A, lda, W, ldw, Y, ldy, ep, nk, (float *)nullptr);
    }
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

// what gemm_dma_kernel assumes: whole k-tiles, 16-byte rows and row starts for its loads and its eight-wide epilogue
bool dma_ok(bool w_u8, int64_t N, int64_t M, const void *A, int64_t lda, const void *W, int64_t ldw, const void *Y, int64_t ldy,
            const GemmEpi &ep) {
    auto a16 = [](const void *p) { return (((uintptr_t)p) & 15) == 0; };
    if ((N % BK) || (M & 7) || (lda & 7) || (ldw & (w_u8 ? 15 : 7)) || (ldy & 7)) return false;
    if (!a16(A) || !a16(W) || !a16(Y)) return false;
    if (w_u8 && (!ep.rx || !ep.mx || !ep.s0 || !ep.s2 || !a16(ep.rx) || !a16(ep.mx))) return false;
    if (!w_u8 && ep.rx) return false;
    if (ep.act == ACT_RESIDUAL || ep.act == ACT_GATED_RESIDUAL)
        if (!ep.res || !a16(ep.res) || (ep.ldres & 7)) return false;
    if (ep.act == ACT_GATED_RESIDUAL)
        if (!ep.gate || !a16(ep.gate) || (ep.ldgate & 7)) return false;
    return true;
}

// Cost model of a direct-to-LDS launch in microseconds, fitted to launches of the 7B shapes (256 to 4096 rows):
// `tiles` tiles of nk k-tiles split c ways run in whole rounds over the 256 CUs; a k-tile step takes 1.75 us with
// the 256 x 256 tile and 0.573 us with the 128 x 128 one (a quarter of the work in a third of the time); every
// round adds its fill, drain and epilogue (10 steps; 4.3 for a split launch, whose epilogue is the reduction pass;
// 12.8 for the small tile, 5.5 where two workgroups per CU overlap); the reduction pass of a split takes 2.5 us
// + 3.6 us per slab and 16 MB of fp32 output, at least 4.5 us.
double dma_cost(int64_t tiles, int nk, int c, bool small_tile, size_t out_bytes) {
    const int64_t rounds = (tiles * c + 255) / 256;
    const double step = small_tile ? 0.573 : 1.75;
    const double extra = small_tile ? (rounds > 1 ? 5.5 : 12.8) : (c > 1 ? 4.3 : 10.0);
    return (double)rounds * (nk / c + extra) * step + (c > 1 ? std::max(4.5, 2.5 + 3.6 * c * (double)out_bytes / (16 << 20)) : 0.0);
}

// the K split (1..8, whole k-tiles, at least 8 per split, slabs within ws_bytes) of least cost
int dma_split(int64_t tiles, int nk, bool small_tile, size_t out_bytes, size_t ws_bytes, double *cost = nullptr) {
    int best = 1;
    double best_cost = 1e30;
    for (int c = 1; c <= 8; ++c) {
        if (nk % c || (c > 1 && nk / c < 8) || (c > 1 && c * out_bytes > ws_bytes)) continue;
        const double k = dma_cost(tiles, nk, c, small_tile, out_bytes);
        if (k < best_cost) { best_cost = k; best = c; }
    }
    if (cost) *cost = best_cost;
    return best;
}

// gemm_dma_kernel.  Fewer than 192 tiles (narrow outputs): the contraction is split over workgroups of the same
// tile until about one workgroup per CU is in flight; slabs and the second pass as in launch_cfg.
template <bool W_U8, int TM, int TN, int NW = 8, int NSTG = 0>
int launch_dma(int64_t T, int64_t N, int64_t M, const rwkv_half *A, int64_t lda, const void *W, int64_t ldw, void *Y,
               int64_t ldy, const GemmEpi &ep, hipStream_t st) {
    constexpr size_t lds = DmaCfg<W_U8, TM, TN, NW, NSTG>::LDS;
    static PerDeviceOnce once;
    bool *attr_done = once.slot();
    if (!attr_done || !*attr_done) {
        hipError_t e = hipFuncSetAttribute((const void *)gemm_dma_kernel<W_U8, false, TM, TN, NW, NSTG>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e == hipSuccess)
            e = hipFuncSetAttribute((const void *)gemm_dma_kernel<W_U8, true, TM, TN, NW, NSTG>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        if (attr_done) *attr_done = true;
    }
    if (!dma_ok(W_U8, N, M, A, lda, W, ldw, Y, ldy, ep)) return RWKV_E_LAYOUT;
    const int64_t tiles = ((T + TM - 1) / TM) * ((M + TN - 1) / TN);
    const int nk = (int)(N / BK);
    int ks = 1;
    if (ep.splitk_ws && (M & 3) == 0) ks = dma_split(tiles, nk, TM < 256, (size_t)T * M * sizeof(float), ep.splitk_bytes);
    if (ks > 1) {
        hipLaunchKernelGGL((gemm_dma_kernel<W_U8, true, TM, TN, NW, NSTG>), dim3((unsigned)tiles, (unsigned)ks), dim3(64 * NW), lds, st, (int)T, (int)N,
                           (int)M, (const h16 *)A, lda, W, ldw, Y, ldy, ep, nk / ks, ep.splitk_ws);
        const int64_t n = T * M;
        const unsigned blocks = (unsigned)((n + 2047) / 2048 < 16384 ? (n + 2047) / 2048 : 16384);
        hipLaunchKernelGGL(splitk_epilogue8_kernel, dim3(blocks), dim3(256), 0, st, (int)T, (int)M, ks, ep.splitk_ws, Y, ldy, ep);
    } else {
        hipLaunchKernelGGL((gemm_dma_kernel<W_U8, false, TM, TN, NW, NSTG>), dim3((unsigned)tiles), dim3(64 * NW), lds, st, (int)T, (int)N, (int)M,
                           (const h16 *)A, lda, W, ldw, Y, ldy, ep, nk, (float *)nullptr);
    }
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

template <bool W_U8>
int launch_pick(int cfg, int64_t T, int64_t N, int64_t M, const rwkv_half *A, int64_t lda, const void *W, int64_t ldw,
                void *Y, int64_t ldy, const GemmEpi &ep, hipStream_t st) {
    switch (cfg) {
        case 3: return launch_cfg<W_U8, 128, 128, 2, 2, 4>(T, N, M, A, lda, W, ldw, Y, ldy, ep, st);
        case 9:
            if constexpr (W_U8) return launch_cfg<true, 256, 256, 4, 4, 2>(T, N, M, A, lda, W, ldw, Y, ldy, ep, st);
            return RWKV_E_DTYPE;
        case 14: return launch_dma<W_U8, 256, 256>(T, N, M, A, lda, W, ldw, Y, ldy, ep, st);
        case 15: return launch_dma<W_U8, 128, 128>(T, N, M, A, lda, W, ldw, Y, ldy, ep, st);
        default: return RWKV_E_DTYPE;
    }
}

// Tile choice (RWKV_GEMM_CFG overrides it for tuning sweeps).
//   14 / 15  operands laid out for 16-byte loads: the direct-to-LDS kernel with 256 x 256 or 128 x 128 tiles,
//            whichever the cost model puts first (large tiles where they fill the chip, small ones at full depth
//            where the large ones would have to split K; small ones when another product runs beside this one)
//    9       uint8 weights otherwise, where 256 x 256 tiles of the register-staged kernel fill the chip: one per CU
//            and round, the last round at least 70 % full
//    3       everything else: 128 x 128 tiles, 4 k-tiles of prefetch
int pick_cfg(int64_t T, int64_t N, int64_t M, bool w_u8, bool alone, bool dma, size_t split_bytes) {
    const char *e = getenv("RWKV_GEMM_CFG");  // tuning override
    if (e && *e) return atoi(e);
    if (!alone) return dma ? 15 : 3;   // a 256 x 256 tile's LDS leaves no room beside it on the CU, two small ones fit
    if (dma) {
        const int nk = (int)(N / BK);
        const size_t out_bytes = (size_t)T * M * sizeof(float), ws = !(M & 3) ? split_bytes : 0;
        double c14, c15;
        dma_split(((T + 255) / 256) * ((M + 255) / 256), nk, false, out_bytes, ws, &c14);
        dma_split(((T + 127) / 128) * ((M + 127) / 128), nk, true, out_bytes, ws, &c15);
        return c14 <= c15 ? 14 : 15;
    }
    const int64_t big = ((T + 255) / 256) * ((M + 255) / 256), rounds = (big + 255) / 256;
    return w_u8 && big * 10 >= rounds * 256 * 7 ? 9 : 3;   // fp16 weight tiles are twice the bytes: the large tile spills
}

}  // namespace

GemmPlan gemm_plan(bool w_u8, int64_t T, int64_t N, int64_t M, const rwkv_half *A, int64_t lda, const void *W,
                   int64_t ldw, const void *Y, int64_t ldy, const GemmEpi &ep) {
    if (skinny_ok(w_u8, T, N, A, lda, W, ldw, ep)) return GemmPlan{0, 0, 0, 1};
    const int cfg = pick_cfg(T, N, M, w_u8, !ep.small_tiles, dma_ok(w_u8, N, M, A, lda, W, ldw, Y, ldy, ep),
                             ep.splitk_ws ? ep.splitk_bytes : 0);
    if (cfg != 14 && cfg != 15) return GemmPlan{1, 0, 0, 1};
    const int tile = cfg == 14 ? 256 : 128;
    const int64_t tiles = ((T + tile - 1) / tile) * ((M + tile - 1) / tile);
    int ks = 1;   // as launch_dma decides it
    if (ep.splitk_ws && (M & 3) == 0) ks = dma_split(tiles, (int)(N / BK), tile < 256, (size_t)T * M * sizeof(float), ep.splitk_bytes);
    return GemmPlan{2, tile, tile, ks};
}

int gemm_launch(bool w_u8, int64_t T, int64_t N, int64_t M, const rwkv_half *A, int64_t lda, const void *W,
                int64_t ldw, void *Y, int64_t ldy, const GemmEpi &ep, hipStream_t st) {
    if (skinny_ok(w_u8, T, N, A, lda, W, ldw, ep)) {
        SkinnyGroup g{};
        g.A[0] = (const h16 *)A; g.W[0] = W; g.Y[0] = Y; g.lda = lda; g.ldw[0] = ldw; g.ldy[0] = ldy; g.M[0] = (int)M; g.ep[0] = ep;
        return skinny_launch(w_u8, 1, T, N, g, st);
    }
    if (narrow_ok(w_u8, T, N, M, A, lda, W, ldw, Y, ldy, ep)) {
        hipLaunchKernelGGL(narrow_kernel, dim3((unsigned)((T + 15) / 16), (unsigned)((M + 15) / 16)), dim3(512), 0, st, (int)T, (int)N,
                           (int)M, (const h16 *)A, lda, (const h16 *)W, ldw, (rwkv_half *)Y, ldy, ep);
        RWKV_LAUNCH_CHECK();
        return RWKV_OK;
    }
    const int cfg = pick_cfg(T, N, M, w_u8, !ep.small_tiles, dma_ok(w_u8, N, M, A, lda, W, ldw, Y, ldy, ep),
                             ep.splitk_ws ? ep.splitk_bytes : 0);
    return w_u8 ? launch_pick<true>(cfg, T, N, M, A, lda, W, ldw, Y, ldy, ep, st)
                : launch_pick<false>(cfg, T, N, M, A, lda, W, ldw, Y, ldy, ep, st);
}

int mm8_prepare_launch(int64_t T, int64_t N, const rwkv_half *x, int64_t ldx, const rwkv_half *ry,
                       const rwkv_half *my, rwkv_half *xs, float *s0, float *s2, hipStream_t st) {
    hipLaunchKernelGGL(mm8_prepare_kernel, dim3((unsigned)T), dim3(256), 0, st, (int)T, (int)N, x, ldx, ry, my, xs, s0, s2);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}


// n (2..4) products [T, N] x [N, M_i] of uint8 or fp16 weights with their own inputs, outputs and epilogues in one
// launch.  uint8 with xs != NULL: x[i] is the unscaled activation and xs[i] / sums[i] (2 T floats) are scratch;
// uint8 with xs == NULL: x[i] is already scaled by ry and sums[i] holds its row sums -- as 2 T totals, or with
// parts > 1 (a multiple of four; direct-to-LDS launches only, see gemm_group_takes_parts) as 2 T floats of scratch
// followed by [T][parts] partial sums of x and [T][parts] of x * my, which the launch adds up in index order.
// Operands laid out for 16-byte loads: the direct-to-LDS kernel, tile size and K split (over splitk_ws,
// RWKV_SPLITK_WS_BYTES of scratch, or NULL) from the cost model; otherwise register-staged 128 x 128 tiles at full depth.
bool gemm_group_takes_parts(bool w_u8, int n, int64_t T, int64_t N, const rwkv_half *const *x, const rwkv_mat *const *mats,
                            void *const *Y) {
    if (!w_u8 || n < 2 || n > 4 || (N % BK)) return false;
    const float one = 0.f;
    bool skinny = true;
    for (int i = 0; i < n; ++i) {
        GemmEpi e{};
        e.mx = mats[i]->mx; e.rx = mats[i]->rx; e.s0 = &one; e.s2 = &one; e.out_dtype = RWKV_DT_F16;
        if (mats[i]->N != N || !dma_ok(true, N, mats[i]->M, x[i], N, mats[i]->w, mats[i]->ld, Y[i], mats[i]->M, e)) return false;
        skinny = skinny && skinny_ok(true, T, N, x[i], N, mats[i]->w, mats[i]->ld, e);
    }
    return !skinny;
}

int gemm_group_launch(bool w_u8, int n, int64_t T, int64_t N, const rwkv_half *const *x, const rwkv_mat *const *mats,
                      void *const *Y, const GemmEpi *eps, rwkv_half *const *xs, float *const *sums, float *splitk_ws,
                      hipStream_t st, int parts) {
    if (n < 2 || n > 4 || (N % BK)) return RWKV_E_SHAPE;
    if (parts > 1 && (xs || !w_u8 || (parts & 3))) return RWKV_E_SHAPE;
    GemmGroup g{};
    g.lda = N;
    const bool prep = w_u8 && xs;
    if (prep) {
        PrepGroup p{};
        for (int i = 0; i < n; ++i) {
            p.x[i] = x[i]; p.ry[i] = mats[i]->ry; p.my[i] = mats[i]->my; p.xs[i] = xs[i]; p.s0[i] = sums[i]; p.s2[i] = sums[i] + T;
        }
        hipLaunchKernelGGL(mm8_prepare_group_kernel, dim3((unsigned)((T + 3) / 4), (unsigned)n), dim3(256), 0, st, (int)T, (int)N, p);
    }
    int64_t tiles = 0, tiles_big = 0, total_big = 0, total_small = 0, out_elems = 0, max_out = 0;
    bool dma = true, m4 = true;
    for (int i = 0; i < n; ++i) {
        if (mats[i]->N != N) return RWKV_E_SHAPE;
        g.A[i] = (const h16 *)(prep ? xs[i] : x[i]);
        g.W[i] = mats[i]->w; g.ldw[i] = mats[i]->ld; g.Y[i] = Y[i]; g.M[i] = (int)mats[i]->M;
        g.ep[i] = eps[i];
        g.ep[i].ldres = g.ep[i].ldgate = mats[i]->M;
        if (w_u8) { g.ep[i].mx = mats[i]->mx; g.ep[i].rx = mats[i]->rx; g.ep[i].s0 = sums[i]; g.ep[i].s2 = sums[i] + T; }
        if (parts > 1) { g.ep[i].parts = parts; g.ep[i].p0 = sums[i] + 2 * T; g.ep[i].p2 = sums[i] + 2 * T + (size_t)T * parts; }
        const int64_t ts = ((T + 127) / 128) * ((mats[i]->M + 127) / 128), tb = ((T + DT - 1) / DT) * ((mats[i]->M + DM - 1) / DM);
        tiles = std::max(tiles, ts);
        tiles_big = std::max(tiles_big, tb);
        total_small += ts;
        total_big += tb;
        out_elems += T * mats[i]->M;
        max_out = std::max<int64_t>(max_out, T * mats[i]->M);
        m4 = m4 && !(mats[i]->M & 3);
        dma = dma && dma_ok(w_u8, N, mats[i]->M, g.A[i], N, g.W[i], g.ldw[i], g.Y[i], mats[i]->M, g.ep[i]);
    }
    {
        bool skinny = true;
        for (int i = 0; i < n; ++i) skinny = skinny && skinny_ok(w_u8, T, N, g.A[i], N, g.W[i], g.ldw[i], g.ep[i]);
        if (skinny) {
            if (parts > 1) return RWKV_E_LAYOUT;
            SkinnyGroup sg{};
            sg.lda = N;
            for (int i = 0; i < n; ++i) {
                sg.A[i] = g.A[i]; sg.W[i] = g.W[i]; sg.Y[i] = g.Y[i]; sg.ldw[i] = g.ldw[i]; sg.ldy[i] = g.M[i]; sg.M[i] = g.M[i];
                sg.ep[i] = g.ep[i];
            }
            return skinny_launch(w_u8, n, T, N, sg, st);
        }
    }
    if (dma) {
        // tile size and K split of least cost, as for a single product
        const int nk = (int)(N / BK);
        const size_t out_bytes = (size_t)out_elems * sizeof(float), ws = splitk_ws && m4 ? RWKV_SPLITK_WS_BYTES : 0;
        double c_big, c_small;
        const int ks_big = dma_split(total_big, nk, false, out_bytes, ws, &c_big);
        const int ks_small = dma_split(total_small, nk, true, out_bytes, ws, &c_small);
        const bool big = c_big <= c_small;
        const int ks = big ? ks_big : ks_small;
        g.nk_split = nk / ks;
        if (ks > 1) {
            float *p = splitk_ws;
            for (int i = 0; i < n; ++i) { g.part[i] = p; p += (size_t)ks * T * mats[i]->M; }
        }
        int rc;
        if (big) rc = w_u8 ? launch_dma_group<true, DT, DM>(g, n, T, N, tiles_big, ks, st) : launch_dma_group<false, DT, DM>(g, n, T, N, tiles_big, ks, st);
        else rc = w_u8 ? launch_dma_group<true, 128, 128>(g, n, T, N, tiles, ks, st) : launch_dma_group<false, 128, 128>(g, n, T, N, tiles, ks, st);
        if (rc) return rc;
        if (ks > 1) {
            const unsigned blocks = (unsigned)std::min<int64_t>((max_out + 2047) / 2048, 16384);
            hipLaunchKernelGGL(splitk_group_epilogue8_kernel, dim3(blocks, (unsigned)n), dim3(256), 0, st, (int)T, ks, g);
        }
        RWKV_LAUNCH_CHECK();
        return RWKV_OK;
    }
    if (parts > 1) return RWKV_E_LAYOUT;   // partial sums only through the direct-to-LDS kernel
    constexpr size_t lds = 2 * (size_t)(128 + 128) * BK * sizeof(h16);
    const dim3 grid((unsigned)tiles, (unsigned)n);
    if (w_u8) hipLaunchKernelGGL((gemm_group_kernel<true, 128, 128, 2, 2, 4>), grid, dim3(256), lds, st, (int)T, (int)N, g);
    else hipLaunchKernelGGL((gemm_group_kernel<false, 128, 128, 2, 2, 4>), grid, dim3(256), lds, st, (int)T, (int)N, g);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

extern "C" size_t rwkv_mm8_seq_workspace(int64_t B, int64_t N) {
    if (B <= 0 || N <= 0) return 0;
    return (((size_t)B * N * 2 + 255) & ~(size_t)255) + (((size_t)B * 8 + 255) & ~(size_t)255) + RWKV_SPLITK_WS_BYTES;
}

// rwkv_mm8_seq_f16 in its two launches: the activation-scaling pass (`reps` < 0), the contraction alone `reps`
// times on the already scaled rows (`reps` > 0), or one of each (`reps` == 0: the product)
static int mm8_seq_parts(int64_t B, int64_t N, int64_t M, const rwkv_half *x, int64_t x_stride, const uint8_t *w,
                         int64_t w_stride_n, int64_t w_stride_m, const rwkv_half *mx, const rwkv_half *rx,
                         const rwkv_half *my, const rwkv_half *ry, rwkv_half *y, int64_t y_stride, void *workspace,
                         size_t workspace_bytes, hipStream_t st, int reps) {
    if (!x || !w || !mx || !rx || !my || !ry || !y || !workspace) return RWKV_E_NULL;
    if (B <= 0 || N <= 0 || M <= 0 || (N % BK) != 0 || B > (1 << 24) || M > (1 << 24)) return RWKV_E_SHAPE;
    if (w_stride_n != 1 || w_stride_m < N || (w_stride_m & 15) || !aligned16(w)) return RWKV_E_LAYOUT;
    if (x_stride < N || (x_stride & 7) || !aligned16(x) || y_stride < M || !aligned16(my) || !aligned16(ry))
        return RWKV_E_LAYOUT;
    if (workspace_bytes < rwkv_mm8_seq_workspace(B, N) || !aligned16(workspace)) return RWKV_E_WORKSPACE;
    rwkv_half *xs = (rwkv_half *)workspace;
    const size_t xs_bytes = ((size_t)B * N * 2 + 255) & ~(size_t)255;
    float *s0 = (float *)((unsigned char *)workspace + xs_bytes);
    float *s2 = s0 + B;
    if (reps <= 0) {
        int rc = mm8_prepare_launch(B, N, x, x_stride, ry, my, xs, s0, s2, st);
        if (rc || reps < 0) return rc;
    }
    GemmEpi ep{};
    ep.mx = mx; ep.rx = rx; ep.s0 = s0; ep.s2 = s2; ep.act = ACT_NONE; ep.out_scale = 1.f; ep.out_dtype = RWKV_DT_F16;
    ep.splitk_ws = (float *)((unsigned char *)workspace + xs_bytes + (((size_t)B * 8 + 255) & ~(size_t)255));
    ep.splitk_bytes = RWKV_SPLITK_WS_BYTES;
    int rc = RWKV_OK;
    for (int r = 0; r < (reps > 0 ? reps : 1) && rc == RWKV_OK; ++r)
        rc = gemm_launch(true, B, N, M, xs, N, w, w_stride_m, y, y_stride, ep, st);
    return rc;
}

extern "C" int rwkv_mm8_seq_f16(int64_t B, int64_t N, int64_t M, const rwkv_half *x, int64_t x_stride,
                                const uint8_t *w, int64_t w_stride_n, int64_t w_stride_m, const rwkv_half *mx,
                                const rwkv_half *rx, const rwkv_half *my, const rwkv_half *ry, rwkv_half *y,
                                int64_t y_stride, void *workspace, size_t workspace_bytes, void *stream) {
    return mm8_seq_parts(B, N, M, x, x_stride, w, w_stride_n, w_stride_m, mx, rx, my, ry, y, y_stride, workspace,
                         workspace_bytes, (hipStream_t)stream, 0);
}

extern "C" int rwkv_mm8_seq_time_kernel(int64_t B, int64_t N, int64_t M, const rwkv_half *x, int64_t x_stride,
                                        const uint8_t *w, int64_t w_stride_n, int64_t w_stride_m,
                                        const rwkv_half *mx, const rwkv_half *rx, const rwkv_half *my,
                                        const rwkv_half *ry, rwkv_half *y, int64_t y_stride, void *workspace,
                                        size_t workspace_bytes, void *stream, int reps, float *ms_per_launch) {
    if (!ms_per_launch) return RWKV_E_NULL;
    if (reps <= 0) return RWKV_E_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    int rc = mm8_seq_parts(B, N, M, x, x_stride, w, w_stride_n, w_stride_m, mx, rx, my, ry, y, y_stride, workspace,
                           workspace_bytes, st, -1);
    if (rc) return rc;
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess) return (int)hipErrorOutOfMemory;
    if (hipEventCreate(&e1) != hipSuccess) { (void)hipEventDestroy(e0); return (int)hipErrorOutOfMemory; }
    (void)hipEventRecord(e0, st);
    rc = mm8_seq_parts(B, N, M, x, x_stride, w, w_stride_n, w_stride_m, mx, rx, my, ry, y, y_stride, workspace,
                       workspace_bytes, st, reps);
    (void)hipEventRecord(e1, st);
    hipError_t e = hipEventSynchronize(e1);
    float ms = 0.f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e != hipSuccess && rc == RWKV_OK) rc = (int)e;
    *ms_per_launch = ms / reps;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return rc;
}

// ---- rwkv_mm8_seq_f16 without a caller workspace ------------------------------------------------------------
// The scratch of the product (the ry-scaled copy of x, its two row sums, split-K slabs) in a file-scope device
// array instead of a workspace argument.  The array's name is only a host-side handle: the device address of each
// GPU's copy comes from hipGetSymbolAddress, once per device, and that pointer is what the kernels get.
constexpr size_t STATIC_XS_BYTES = (size_t)8 << 20;       // B * N <= 4 Mi elements
constexpr size_t STATIC_SUMS_BYTES = (size_t)64 << 10;    // B <= 8192
constexpr size_t STATIC_SPLITK_BYTES = (size_t)16 << 20;  // the K split is limited to slabs that fit here
constexpr size_t STATIC_SCRATCH_BYTES = STATIC_XS_BYTES + STATIC_SUMS_BYTES + STATIC_SPLITK_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

constexpr int STATIC_MAX_DEVICES = 64;
static void *g_scratch_ptr[STATIC_MAX_DEVICES];
static std::mutex g_scratch_mutex;

// device address of the current device's copy of `scratch` (looked up on the first call on that device)
static int static_scratch(unsigned char **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= STATIC_MAX_DEVICES) return RWKV_E_SHAPE;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return RWKV_E_NULL;
        g_scratch_ptr[dev] = p;
    }
    *out = (unsigned char *)g_scratch_ptr[dev];
    return RWKV_OK;
}

extern "C" size_t rwkv_mm8_seq_static_max_elems(void) { return STATIC_XS_BYTES / 2; }
extern "C" size_t rwkv_mm8_seq_static_max_rows(void) { return STATIC_SUMS_BYTES / 8; }

extern "C" int rwkv_mm8_seq_f16_static(int64_t B, int64_t N, int64_t M, const rwkv_half *x, int64_t x_stride,
                                       const uint8_t *w, int64_t w_stride_n, int64_t w_stride_m, const rwkv_half *mx,
                                       const rwkv_half *rx, const rwkv_half *my, const rwkv_half *ry, rwkv_half *y,
                                       int64_t y_stride, void *stream) {
    if (!x || !w || !mx || !rx || !my || !ry || !y) return RWKV_E_NULL;
    if (B <= 0 || N <= 0 || M <= 0 || (N % BK) != 0 || B > (1 << 24) || M > (1 << 24)) return RWKV_E_SHAPE;
    if (w_stride_n != 1 || w_stride_m < N || (w_stride_m & 15) || !aligned16(w)) return RWKV_E_LAYOUT;
    if (x_stride < N || (x_stride & 7) || !aligned16(x) || y_stride < M || !aligned16(my) || !aligned16(ry))
        return RWKV_E_LAYOUT;
    if ((size_t)B * (size_t)N * 2 > STATIC_XS_BYTES || (size_t)B * 8 > STATIC_SUMS_BYTES) return RWKV_E_SCRATCH;
    unsigned char *base = nullptr;
    int rc = static_scratch(&base);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    rwkv_half *xs = (rwkv_half *)base;
    float *s0 = (float *)(base + STATIC_XS_BYTES);
    float *s2 = s0 + B;
    // every row of xs / s0 / s2 and every slab element the product reads is written by this call first:
    // nothing in the array has to start at zero
    rc = mm8_prepare_launch(B, N, x, x_stride, ry, my, xs, s0, s2, st);
    if (rc) return rc;
    GemmEpi ep{};
    ep.mx = mx; ep.rx = rx; ep.s0 = s0; ep.s2 = s2; ep.act = ACT_NONE; ep.out_scale = 1.f; ep.out_dtype = RWKV_DT_F16;
    ep.splitk_ws = (float *)(base + STATIC_XS_BYTES + STATIC_SUMS_BYTES);
    ep.splitk_bytes = STATIC_SPLITK_BYTES;
    return gemm_launch(true, B, N, M, xs, N, w, w_stride_m, y, y_stride, ep, st);
}

extern "C" int rwkv_gemm_f16(int64_t B, int64_t N, int64_t M, const rwkv_half *a, int64_t a_stride,
                             const rwkv_half *b, int64_t b_stride_n, int64_t b_stride_m, void *c, int64_t c_stride,
                             int c_dtype, void *stream) {
    if (!a || !b || !c) return RWKV_E_NULL;
    if (B <= 0 || N <= 0 || M <= 0 || (N & 7) || B > (1 << 24) || M > (1 << 24)) return RWKV_E_SHAPE;
    if (c_dtype != RWKV_DT_F16 && c_dtype != RWKV_DT_F32) return RWKV_E_DTYPE;
    if (b_stride_n != 1 || b_stride_m < N || (b_stride_m & 7) || !aligned16(b)) return RWKV_E_LAYOUT;
    if (a_stride < N || (a_stride & 7) || !aligned16(a) || c_stride < M) return RWKV_E_LAYOUT;
    hipStream_t st = (hipStream_t)stream;
    if (B == 1) {
        if (N > 32768) return RWKV_E_SHAPE;
        return gemv_f16_launch(N, M, a, b, b_stride_m, c, c_dtype, st);
    }
    if (N % BK) return RWKV_E_SHAPE;
    GemmEpi ep{};
    ep.act = ACT_NONE; ep.out_scale = 1.f; ep.out_dtype = c_dtype; ep.raw_f32 = (c_dtype == RWKV_DT_F32);
    return gemm_launch(false, B, N, M, a, a_stride, b, b_stride_m, c, c_stride, ep, st);
}

extern "C" int rwkv_gemm_f16_batched(int64_t batch, int64_t B, int64_t N, int64_t M, const rwkv_half *a, int64_t a_stride,
                                     int64_t a_batch_stride, const rwkv_half *b, int64_t b_stride_n, int64_t b_stride_m,
                                     int64_t b_batch_stride, void *c, int64_t c_stride, int64_t c_batch_stride, int c_dtype,
                                     void *stream) {
    if (batch <= 0 || batch > (1 << 20)) return RWKV_E_SHAPE;
    if (!a || !b || !c) return RWKV_E_NULL;
    if (c_dtype != RWKV_DT_F16 && c_dtype != RWKV_DT_F32) return RWKV_E_DTYPE;
    // every product of the batch must itself be acceptable: 16-byte aligned operands
    if ((a_batch_stride & 7) || (b_batch_stride & 7) || a_batch_stride < 0 || b_batch_stride < 0 || c_batch_stride < 0)
        return RWKV_E_LAYOUT;
    const size_t csz = c_dtype == RWKV_DT_F16 ? 2 : 4;
    for (int64_t i = 0; i < batch; ++i) {
        const int rc = rwkv_gemm_f16(B, N, M, a + i * a_batch_stride, a_stride, b + i * b_batch_stride, b_stride_n, b_stride_m,
                                     (char *)c + (size_t)(i * c_batch_stride) * csz, c_stride, c_dtype, stream);
        if (rc) return rc;
    }
    return RWKV_OK;
}
