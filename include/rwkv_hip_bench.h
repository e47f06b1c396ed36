/*
 * Measurement aids of librwkv_hip.so: blocking entry points that time the one-token step of
 * rwkv_v4_forward_one and the contraction kernel of rwkv_mm8_seq_f16 (include/rwkv_hip.h) with HIP events on
 * the stream the kernels run on.  They replace
 * nothing in the reference and are not part of the product interface: bench.py is their only caller.
 */
#ifndef RWKV_HIP_BENCH_H
#define RWKV_HIP_BENCH_H

#include "rwkv_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Measurement aid: the same step as rwkv_v4_forward_one with a HIP event recorded on `stream`
 * around every kernel launch.  Blocks until the step has finished and writes the elapsed
 * milliseconds of the 4 * n_layer + 1 launches to ms[] in launch order: per layer (time-mix
 * k/v/r + WKV, time-mix output, channel-mix r/k, channel-mix value), then the head.
 * Not capturable (it synchronises). */
int rwkv_v4_profile_one(const rwkv_v4_model *m, const rwkv_v4_layer_state *states, const int32_t *token,
                        float *logits, void *workspace, size_t workspace_bytes, void *stream,
                        float *ms, int64_t n_ms);

/* Measurement aid: launches ONE phase of the step (0 time-mix k/v/r + WKV, 1 time-mix output,
 * 2 channel-mix r/k, 3 channel-mix value: once per layer, each layer streaming its own weights;
 * 4 head) `reps` times back to back between two HIP events on `stream`, blocks, and returns the
 * mean duration of one launch in milliseconds.  Results written to the state / logits are
 * meaningless: pass a scratch state. */
int rwkv_v4_time_phase(const rwkv_v4_model *m, const rwkv_v4_layer_state *states, const int32_t *token,
                       float *logits, void *workspace, size_t workspace_bytes, void *stream, int phase,
                       int reps, float *ms_per_launch);

/* Measurement aid: the arguments of rwkv_mm8_seq_f16.  Runs its activation-scaling pass once, then the
 * contraction kernel alone `reps` times back to back on the scaled rows between two HIP events on `stream`,
 * blocks, and returns the mean duration of one contraction launch in milliseconds (both launches of a product
 * whose K is split).  y holds the product afterwards. */
int rwkv_mm8_seq_time_kernel(int64_t B, int64_t N, int64_t M, const rwkv_half *x, int64_t x_stride,
                             const uint8_t *w, int64_t w_stride_n, int64_t w_stride_m, const rwkv_half *mx,
                             const rwkv_half *rx, const rwkv_half *my, const rwkv_half *ry, rwkv_half *y,
                             int64_t y_stride, void *workspace, size_t workspace_bytes, void *stream, int reps,
                             float *ms_per_launch);

#ifdef __cplusplus
}
#endif
#endif /* RWKV_HIP_BENCH_H */
