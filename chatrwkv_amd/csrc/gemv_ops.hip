// Operator-level GEMV entry points: rwkv_mm8_one_f16 and the B == 1 path of rwkv_gemm_f16.
#include "gemv_core.h"
#include "kernels.h"

namespace {

constexpr int GEMV_THREADS = 256;

// y[m] = x @ W'[:, m] for uint8 weights.  Every workgroup rebuilds the scaled activation
// vector in LDS (N is a few thousand elements, served from L2), then its waves stream rows.
template <int R, int U>
__global__ __launch_bounds__(GEMV_THREADS) void mm8_one_kernel(
    int N, int M, const rwkv_half *__restrict__ x, const uint8_t *__restrict__ w, int64_t ldw,
    const rwkv_half *__restrict__ mx, const rwkv_half *__restrict__ rx, const rwkv_half *__restrict__ my,
    const rwkv_half *__restrict__ ry, void *__restrict__ y, int y_dtype) {
    extern __shared__ __align__(16) unsigned char smem[];
    h16 *xs = (h16 *)smem;
    __shared__ float red[GEMV_THREADS / 64];
    const int nseg = N >> 4;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f;
    for (int j = threadIdx.x; j < N; j += blockDim.x) {
        const float xv = h2f(x[j]);
        const h16 sc = (h16)(xv * h2f(ry[j]));
        xs[xs_slot(j, nseg)] = sc;
        s0 += xv;
        s1 += (float)sc;
        s2 += xv * h2f(my[j]);
    }
    VecSums S;
    S.s0 = block_sum(s0, red);
    S.s1 = block_sum(s1, red);
    S.s2 = block_sum(s2, red);
    __syncthreads();

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nwaves = gridDim.x * (GEMV_THREADS / 64);
    const int ngroups = (M + R - 1) / R;
    for (int g = blockIdx.x * (GEMV_THREADS / 64) + wave; g < ngroups; g += nwaves) {
        const uint8_t *rows[R];
        const h16 *xv[R];
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int m = min(g * R + r, M - 1);
            rows[r] = w + (size_t)m * ldw;
            xv[r] = xs;
            acc[r] = 0.f;
        }
        wave_rows_dot_u8<R, U>(rows, xv, nseg, acc);
        if (lane < R) {
            float a = acc[0];
#pragma unroll
            for (int r = 1; r < R; ++r) a = (lane == r) ? acc[r] : a;
            const int m = g * R + lane;
            if (m < M) {
                const float v = mm8_finish(a, S, h2f(rx[m]), h2f(mx[m]));
                if (y_dtype == RWKV_DT_F32)
                    ((float *)y)[m] = v;
                else
                    ((rwkv_half *)y)[m] = f2h(v);
            }
        }
    }
}

template <int R, int U>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_f16_kernel(
    int N, int M, const rwkv_half *__restrict__ x, const h16 *__restrict__ w, int64_t ldw,
    void *__restrict__ y, int y_dtype) {
    extern __shared__ __align__(16) unsigned char smem[];
    h16 *xs = (h16 *)smem;
    for (int j = threadIdx.x; j < N; j += blockDim.x) xs[j] = __builtin_bit_cast(h16, x[j]);
    __syncthreads();
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nwaves = gridDim.x * (GEMV_THREADS / 64);
    const int ngroups = (M + R - 1) / R;
    for (int g = blockIdx.x * (GEMV_THREADS / 64) + wave; g < ngroups; g += nwaves) {
        const h16 *rows[R];
        const h16 *xv[R];
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int m = min(g * R + r, M - 1);
            rows[r] = w + (size_t)m * ldw;
            xv[r] = xs;
            acc[r] = 0.f;
        }
        wave_rows_dot_f16<R, U>(rows, xv, N >> 3, acc);
        if (lane < R) {
            float a = acc[0];
#pragma unroll
            for (int r = 1; r < R; ++r) a = (lane == r) ? acc[r] : a;
            const int m = g * R + lane;
            if (m < M) {
                if (y_dtype == RWKV_DT_F32)
                    ((float *)y)[m] = a;
                else
                    ((rwkv_half *)y)[m] = f2h(a);
            }
        }
    }
}

int pick_grid(int64_t M, int R) {
    // 256 CUs; up to 8 workgroups of 4 waves per CU are resident.  Use enough waves that every
    // wave gets at least one row group, but no more than 2048 workgroups.
    const int64_t groups = (M + R - 1) / R;
    int64_t blocks = (groups + 3) / 4;
    if (blocks > 2048) blocks = 2048;
    if (blocks < 1) blocks = 1;
    return (int)blocks;
}

}  // namespace

int gemv_f16_launch(int64_t N, int64_t M, const rwkv_half *x, const rwkv_half *w, int64_t ldw, void *y,
                    int y_dtype, hipStream_t st) {
    const size_t lds = (size_t)N * 2;
    if (M >= 16384) {
        hipLaunchKernelGGL((gemv_f16_kernel<2, 4>), dim3(pick_grid(M, 2)), dim3(GEMV_THREADS), lds, st, (int)N,
                           (int)M, x, (const h16 *)w, ldw, y, y_dtype);
    } else {
        hipLaunchKernelGGL((gemv_f16_kernel<1, 8>), dim3(pick_grid(M, 1)), dim3(GEMV_THREADS), lds, st, (int)N,
                           (int)M, x, (const h16 *)w, ldw, y, y_dtype);
    }
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

extern "C" int rwkv_mm8_one_f16(int64_t N, int64_t M, const rwkv_half *x, const uint8_t *w, int64_t w_stride_n,
                                int64_t w_stride_m, const rwkv_half *mx, const rwkv_half *rx,
                                const rwkv_half *my, const rwkv_half *ry, void *y, int y_dtype, void *stream) {
    if (!x || !w || !mx || !rx || !my || !ry || !y) return RWKV_E_NULL;
    if (N <= 0 || M <= 0 || (N & 15) || N > 32768 || M > (1 << 30)) return RWKV_E_SHAPE;
    if (y_dtype != RWKV_DT_F16 && y_dtype != RWKV_DT_F32) return RWKV_E_DTYPE;
    if (w_stride_n != 1 || w_stride_m < N || (w_stride_m & 15) || !aligned16(w)) return RWKV_E_LAYOUT;
    hipStream_t st = (hipStream_t)stream;
    const size_t lds = (size_t)N * 2;
    if (M >= 16384) {
        hipLaunchKernelGGL((mm8_one_kernel<4, 2>), dim3(pick_grid(M, 4)), dim3(GEMV_THREADS), lds, st, (int)N,
                           (int)M, x, w, w_stride_m, mx, rx, my, ry, y, y_dtype);
    } else if (N >= 8192) {
        hipLaunchKernelGGL((mm8_one_kernel<1, 8>), dim3(pick_grid(M, 1)), dim3(GEMV_THREADS), lds, st, (int)N,
                           (int)M, x, w, w_stride_m, mx, rx, my, ry, y, y_dtype);
    } else {
        hipLaunchKernelGGL((mm8_one_kernel<1, 4>), dim3(pick_grid(M, 1)), dim3(GEMV_THREADS), lds, st, (int)N,
                           (int)M, x, w, w_stride_m, mx, rx, my, ry, y, y_dtype);
    }
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}
