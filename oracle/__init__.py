"""CPU oracle for the quantized RWKV inference hot path.  TEST INFRASTRUCTURE ONLY.

This package restates, in numpy, the arithmetic of the reference path
``RWKV(model, strategy).forward(tokens, state)``
(rwkv_pip_package/src/rwkv/model.py:612-1677 and the kernels under
rwkv_pip_package/src/rwkv/cuda/).  It exists to check the HIP path and to be
timed as the CPU baseline.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it; the product package
``chatrwkv_amd`` never does and fails loudly when its HIP library is missing.

Modules
  quant.py   uint8 quantizer + dequantisation          (model.py:818-847, 91-97)
  ops.py     LayerNorm/GroupNorm, mm8, WKV v4/v5/v6     (model.py:984-1340, cuda/*.cu)
  model.py   checkpoint conversion + forward            (model.py:613-903, 1443-1677)
  sampling.py  sampling step after the path           (utils.py:55-88, 103-123)
  model_v7.py  RWKV-7 (RWKV_x070) loading + forward     (model.py:223-608, cuda/rwkv7.cu)

How each function is pinned (what a wrong sign / index / dropped term would trip):
  sampling.*           the reference's own draws for seeded numpy generators
                       (tests/golden/sampler.npz) + hand-worked cuts, ties, penalties.
  quantize_u8          golden vectors written by the reference's own loader
                       (tests/golden/quant_*.npz) + invariants (0 and 255 in
                       every row and column, reconstruction bound).
  mm8 / dequant        fp64 ``x @ W'`` library matmul; factorised identity.
  wkv4_*               O(T^2) closed form in fp64; zero-state T=1 => wkv = v;
                       golden end-to-end logits + state from the reference.
  wkv5/6 recurrences   O(T^2) closed form in fp64; v5 parallel form vs recurrent
                       form; non-symmetric state for the [h][key][value] layout;
                       golden end-to-end logits + state from the reference.
  layer_norm/group_norm  torch CPU library routines.
  forward (all versions) golden logits and final state from the reference's CPU
                       path ('cpu fp32i8', 'cpu fp32'); chunk invariance.
  model_v7.*           golden logits and final states from the reference's RWKV_x070 on
                       the CPU under 'cpu fp32' AND 'cpu fp16' (the latter pins the fp16
                       rounding points, tests/golden/e2e_v7_*.npz); the two restatements
                       of the recurrence against each other, against a scalar loop and
                       against the closed form of the a = 0 special case.
Where the half-precision path rounds is pinned by the reference itself: its pure-torch
functions run on the CPU under 'cpu fp16' (tests/golden/e2e_*_cpu_fp16.npz, RWKV-4 to 6 and
RWKV-7, incl. 8-layer models where the rescale acts); the oracle's 'cpu fp16' mode restates
that run and its 'cuda fp16' emulation stays within one half-precision ulp of it.  What
cannot be executed anywhere in this build (it needs nvcc and an NVIDIA GPU) and is therefore
restated from the reference text only -- "parity unpinned" -- is the arithmetic specific to
the reference's native CUDA library: the fp32 evaluation order inside kernel_mm_seq_fp16i8 /
kernel_mm_one_fp16i8 with their fp16 outputs (cuda/operators.cu:116-246, model.py:63-86) and
gemm_fp16_cublas writing fp32 without an intermediate fp16 rounding
(cuda/gemm_fp16_cublas.cpp:31-33); the values they compute are pinned in fp32 by the
'cpu fp32i8' goldens.
"""
