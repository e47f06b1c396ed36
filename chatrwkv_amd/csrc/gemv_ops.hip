// Operator-level GEMV entry points: rwkv_mm8_one_f16 and the one-row path of rwkv_gemm_f16.  Both run the
// streaming vector kernel of the one-token model path (vec_kernel: ry scaling and the row sums in its
// prologue, rounding in its epilogue).
#include "decode_kernels.h"

namespace {

// x [N] @ matrix -> y [M]; y_dtype fp32 stores the raw sum, fp16 the rounded one.
int vec_op_launch(bool u8, int64_t N, int64_t M, const rwkv_half *x, const MatDev &mat, void *y, int y_dtype, hipStream_t st) {
    VecArgs a{};
    a.vin = x; a.N = (int)N; a.M = (int)M; a.mat = mat;
    a.act = y_dtype == RWKV_DT_F32 ? VACT_F32 : VACT_F16;
    a.out = y; a.out_scale = 1.f;
    vec_launch(u8, a, num_cu(), st);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

}  // namespace

int gemv_f16_launch(int64_t N, int64_t M, const rwkv_half *x, const rwkv_half *w, int64_t ldw, void *y,
                    int y_dtype, hipStream_t st) {
    if ((N & 7) || N > 8 * VP * DTHREADS || !aligned16(x)) return RWKV_E_SHAPE;
    return vec_op_launch(false, N, M, x, MatDev{w, ldw, nullptr, nullptr, nullptr, nullptr}, y, y_dtype, st);
}

extern "C" int rwkv_mm8_one_f16(int64_t N, int64_t M, const rwkv_half *x, const uint8_t *w, int64_t w_stride_n,
                                int64_t w_stride_m, const rwkv_half *mx, const rwkv_half *rx,
                                const rwkv_half *my, const rwkv_half *ry, void *y, int y_dtype, void *stream) {
    if (!x || !w || !mx || !rx || !my || !ry || !y) return RWKV_E_NULL;
    if (N <= 0 || M <= 0 || (N & 15) || N > 8 * VP * DTHREADS || M > (1 << 30)) return RWKV_E_SHAPE;
    if (y_dtype != RWKV_DT_F16 && y_dtype != RWKV_DT_F32) return RWKV_E_DTYPE;
    if (w_stride_n != 1 || w_stride_m < N || (w_stride_m & 15) || !aligned16(w) || !aligned16(x) || !aligned16(my) ||
        !aligned16(ry))
        return RWKV_E_LAYOUT;
    return vec_op_launch(true, N, M, x, MatDev{w, w_stride_m, mx, rx, my, ry}, y, y_dtype, (hipStream_t)stream);
}
