"""Headline benchmark: RWKV-4 7B-shape 'cuda fp16i8', batch 1, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--shape v4-7b] [--no-cpu]

Workload (the headline configuration): random-init 32-layer / n_embd 4096 / ffn 16384 / vocab
50277 model, prefill of 1024 uniform-random tokens in one call, then greedy decode.  A "step"
is one decoded token (one pass of forward([token], state)); W untimed steps, then exactly K
timed steps with the next token taken on the device (rwkv_greedy_token: argmax of the logits) so the loop has no host
synchronisation; the same K steps are also timed with a host sync per token.

One JSON line is printed:
  value / ms_per_step   decode tokens/s (device-token loop) and ms per token
  roofline              the dominant decode kernel (channel-mix receptance+key GEMV): algorithmic
                        bytes per launch / mean launch duration, HIP events around 8 x n_layer
                        back-to-back launches over all layers' weights (rwkv_v4_time_phase), against
                        the 8 TB/s HBM peak
  decode_hbm            whole-step figure: uint8 weight bytes per token x tokens/s / 8 TB/s
  prefill               prefill tokens/s and the MFMA fraction of the whole prefill
  isolated_mm8_op       the dequant-matmul operator alone at the 7B shapes: mm8_one GB/s, mm8_seq TFLOP/s
  prefill_roofline      the prefill contraction kernel alone on the model's largest matrix shape: 2 T N M flops /
                        mean launch duration (HIP events around 20 launches, rwkv_mm8_seq_time_kernel), against
                        the 2.5 PFLOP/s dense fp16 MFMA peak; "with_scaling_pass" = the whole rwkv_mm8_seq_f16
  cpu_baseline          the oracle's 'cpu fp32i8' path (numpy port of the reference's CPU arithmetic) timed on this
                        host on configs[0] (169M shape, 128-token prefill + 32 greedy steps, all BLAS threads)
  cpu_baseline_layer_sample   the same path on one layer + head of the benchmarked shape, extrapolated per token
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12      # bytes/s, MI355X HBM3E
# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by a 1 GiB copy
# kernel: x2.0 / x1.0).  Counter figures, not read in this run: TRAFFIC_SOURCE has the commands and the table, and
# every roofline object names it next to the number so that a stale value can be told from a fresh one.
TRAFFIC_SOURCE = "profiles/decode_7b_fp16i8_hbm_traffic.md"
# (bytes read, bytes written) per launch as that profile lists them
TRAFFIC_READ_WRITTEN = {("v4-7b", "cuda fp16i8", 32, "ffn_rk"): (85079450, 49254),
                        ("v4-7b", "cuda fp16i8", 32, "att_kvr_wkv"): (52175258, 65536),
                        # the prefill contraction [1024 x 4096] x [4096 x 16384], uint8 weights, 256 x 256 tiles
                        ("gemm", 1024, 4096, 16384, True): (134548480, 33554432)}
MEASURED_TRAFFIC = {k: r + w for k, (r, w) in TRAFFIC_READ_WRITTEN.items()}
MFMA_F16_PEAK = 2.5e15  # flop/s dense fp16


def u8_weight_bytes(L, C, F, V, version=4):
    """uint8 matrix bytes one decoded token streams: v4/v5 layers have 5 C x C matrices (v5.1+ a gate: 6),
    v6 has 6; all have the two C x F channel-mix matrices; plus the head."""
    per_layer = (5 if version < 5.1 else 6) * C * C + 2 * C * F
    return L * per_layer + C * V


def _cpu_info():
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] + [1])
    except Exception:
        threads = os.cpu_count() or 1
    return model, int(threads)


def cpu_baseline_cfg0():
    """The reference's 'cpu fp32i8' path (oracle restatement: fp32 activations, every product dequantises its whole
    uint8 matrix first, model.py:91-97) on BASELINE.json configs[0]: RWKV-4 169M shape, prefill of 128 tokens in
    one call, then 32 greedy one-token steps, all BLAS threads of this host.  One warm-up pass (prefill + 2
    steps), then the prefill three times (median) and the 32 steps once (median per step): about 20 s of CPU work.  Converted weights are random bytes and scales (the path's speed
    does not depend on the values; the arithmetic is pinned by tests/golden/e2e_v4_169m_cpu_fp32i8.npz)."""
    import numpy as np
    from chatrwkv_amd import synth
    from oracle.model import OracleRWKV
    _, L, C, F, V = synth.SHAPES["v4-169m"]
    o = OracleRWKV.random_converted_v4(L, C, F, V, seed=0, emb_rows=V)
    toks = synth.random_tokens(128, V, seed=0)

    out, st = o.forward(toks, None)
    for _ in range(2):
        out, st = o.forward([int(out.argmax())], st)
    pre = []
    for _ in range(3):
        a = time.perf_counter()
        out, st = o.forward(toks, None)
        pre.append(time.perf_counter() - a)
    dec = []
    for _ in range(32):
        a = time.perf_counter()
        out, st = o.forward([int(out.argmax())], st)
        dec.append(time.perf_counter() - a)
    t_pre, t_dec = float(np.median(pre)), float(np.median(dec))
    model, threads = _cpu_info()
    return {
        "value": 1.0 / t_dec, "unit": "tok/s", "cores": threads, "kind": "port",
        "sample": (f"BASELINE.json configs[0]: RWKV-4 169M shape ({L} layers, n_embd {C}) 'cpu fp32i8', prefill 128 tokens in "
                   f"one call (median of 3) + 32 greedy steps (median per step) after a warm-up pass, numpy oracle; value = decode tok/s"),
        "prefill_tok_s": 128.0 / t_pre, "decode_tok_s": 1.0 / t_dec, "cpu_model": model,
        "os_cpu_count": os.cpu_count(), "blas_threads": threads,
    }


def cpu_baseline(shape, budget_s=25.0):
    """Oracle 'cpu fp32i8' (dequantise the whole matrix per call, fp32 matvec: the reference's
    CPU path) on a bounded sample: ONE layer of the named shape plus the head, a few tokens;
    per-token time of the full model = n_layer * t_layer + t_head."""
    import numpy as np
    from chatrwkv_amd import synth
    from oracle import ops as oops
    from oracle.model import OracleRWKV
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] + [1])
    except Exception:
        threads = os.cpu_count() or 1
    version, L, C, F, V = synth.SHAPES[shape]
    t0 = time.perf_counter()
    # converted weights filled with random bytes/scales: the CPU path's speed does not depend on values
    o = OracleRWKV.random_converted_v4(1, C, F, V, seed=0)
    setup = time.perf_counter() - t0
    st = o.init_state()
    x = o.w["emb.weight"][[1]].astype(np.float32)
    # warm-up token, then timed tokens through the single layer and through the head
    tl, th = [], []
    deadline = time.perf_counter() + budget_s
    for it in range(5):
        a = time.perf_counter()
        y, st[0], st[1], st[2], st[3] = o._att_v4(x, st[0], st[1], st[2], st[3], 0)
        y, st[4] = o._ffn(y, st[4], 0)
        b = time.perf_counter()
        z = oops.layer_norm(y, o.w["ln_out.weight"], o.w["ln_out.bias"])
        z = oops.matmul(z, o.mat("head.weight"), o.atype, cache=False)
        c = time.perf_counter()
        if it > 0:
            tl.append(b - a)
            th.append(c - b)
        if time.perf_counter() > deadline and len(tl) >= 2:
            break
    t_layer, t_head = float(np.median(tl)), float(np.median(th))
    per_token = L * t_layer + t_head
    return {
        "value": 1.0 / per_token, "unit": "tok/s", "cores": int(threads), "kind": "port",
        "sample": (f"{shape}: {len(tl)} tokens through 1 of {L} layers + head, numpy oracle 'cpu fp32i8' "
                   f"(whole-matrix dequantisation per call, single-threaded elementwise + {threads}-thread BLAS); "
                   f"t_layer {t_layer * 1e3:.0f} ms, t_head {t_head * 1e3:.0f} ms, "
                   f"per token = {L} x t_layer + t_head = {per_token:.2f} s; setup {setup:.0f} s"),
    }


SPINUP_S = 1.0


def spin_up(fn, seconds, sync_every=1):
    """Runs fn() untimed for `seconds` (host clock), synchronising every `sync_every` calls so that the host does
    not run ahead of the device; returns with the device idle for no longer than that last synchronisation."""
    import torch
    t0 = time.perf_counter()
    i = 0
    while time.perf_counter() - t0 < seconds:
        fn()
        i += 1
        if i % sync_every == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    return i


def gemm_roofline(T, N, M, u8, reps=20):
    """The prefill contraction kernel alone on the model's largest matrix shape (channel-mix key,
    [T, N] x [N, M]), launched through the C ABI and timed with two events on the stream it is launched on:
    algorithmic flops 2 T N M over the mean launch time against the dense fp16 MFMA peak.  With uint8 weights the
    kernel is timed on rows that rwkv_mm8_seq_f16's activation-scaling pass has already scaled
    (rwkv_mm8_seq_time_kernel), which is the duration a kernel trace reports for it; the whole operator, scaling
    pass included, is timed beside it ("with_scaling_pass")."""
    import ctypes
    import torch
    from chatrwkv_amd import lib
    L = lib.load()
    dev = "cuda:0"
    x = torch.randn(T, N, device=dev).half()
    y = torch.empty(T, M, device=dev, dtype=torch.float16)
    st = torch.cuda.current_stream().cuda_stream
    flops = 2.0 * T * N * M

    def timed(run):
        for _ in range(3):
            run()
        spin_up(run, min(SPINUP_S, 0.5), sync_every=32)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            run()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / reps

    extra = {}
    if u8:
        w = torch.randint(0, 256, (M, N), dtype=torch.uint8, device=dev)
        mx = torch.randn(M, device=dev).half(); rx = (torch.rand(M, device=dev) * 0.01).half()
        my = torch.randn(N, device=dev).half(); ry = (torch.rand(N, device=dev) * 0.06).half()
        nbytes = L.rwkv_mm8_seq_workspace(T, N)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        args = (T, N, M, x.data_ptr(), N, w.data_ptr(), 1, N, mx.data_ptr(), rx.data_ptr(), my.data_ptr(),
                ry.data_ptr(), y.data_ptr(), M, ws.data_ptr(), nbytes, st)

        def run():
            lib.check(L.rwkv_mm8_seq_f16(*args), "rwkv_mm8_seq_f16")
        t_op = timed(run)
        ms = ctypes.c_float(0.0)
        lib.check(L.rwkv_mm8_seq_time_kernel(*args, reps, ctypes.byref(ms)), "rwkv_mm8_seq_time_kernel")
        t = ms.value * 1e-3
        name = "gemm_dma_kernel<uint8 weights> (direct-to-LDS loads; 256x256 or 128x128 tile by the launch cost model)"
        extra = {"with_scaling_pass": {"kernel": "mm8_prepare_kernel + " + name.split(" (")[0],
                                       "ms_per_call": t_op * 1e3, "achieved": flops / t_op / 1e12,
                                       "frac": flops / t_op / MFMA_F16_PEAK}}
    else:
        w = torch.randn(M, N, device=dev).half()

        def run():
            lib.check(L.rwkv_gemm_f16(T, N, M, x.data_ptr(), N, w.data_ptr(), 1, N, y.data_ptr(), M, lib.RWKV_DT_F16, st),
                      "rwkv_gemm_f16")
        name = "gemm_dma_kernel<fp16 weights> (direct-to-LDS loads; 256x256 or 128x128 tile by the launch cost model)"
        t = timed(run)
    return {"bound": "mfma", "kernel": f"{name}, [{T} x {N}] x [{N} x {M}]", "achieved": flops / t / 1e12,
            "peak": MFMA_F16_PEAK / 1e12, "unit": "TFLOP/s", "frac": flops / t / MFMA_F16_PEAK,
            "scope": "contraction kernel alone (the duration a kernel trace reports for it); the operator with its "
                     "activation-scaling pass is under with_scaling_pass",
            "inputs": "synthetic: uniform random uint8 weights and random fp16 scale vectors rather than quantizer "
                      "output, one 67 MB weight copy reused by every launch (resident in the memory-side cache); "
                      "neither matters to an MFMA-bound duration",
            "traffic": MEASURED_TRAFFIC.get(("gemm", T, N, M, bool(u8))),
            "traffic_source": TRAFFIC_SOURCE if ("gemm", T, N, M, bool(u8)) in MEASURED_TRAFFIC else None,
            "flops_per_launch": flops, "ms_per_launch": t * 1e3, **extra}


def isolated_mm8(reps=40):
    """The isolated uint8 dequant-matmul operator at the 7B shapes (uint8 [4096 x 4096] and [4096 x 16384] with
    fp16 scales, fp16 x ~ N(0, 1)): mm8_one as GB/s of weight bytes (each call streams a different copy of the
    matrix, more than the 256 MB memory-side cache in total) and mm8_seq at 1024 rows as TFLOP/s, both
    through the C ABI and timed with events on the launch stream."""
    import torch
    from chatrwkv_amd import lib
    L = lib.load()
    dev = "cuda:0"
    st = torch.cuda.current_stream().cuda_stream
    out = {}
    for N, M in ((4096, 4096), (4096, 16384)):
        ncopy = max(2, (640 << 20) // (N * M))
        w = torch.randint(0, 256, (ncopy, M, N), dtype=torch.uint8, device=dev)
        mx = torch.randn(M, device=dev).half(); rx = (torch.rand(M, device=dev) * 0.01).half()
        my = torch.randn(N, device=dev).half(); ry = (torch.rand(N, device=dev) * 0.06).half()
        x1 = torch.randn(N, device=dev).half()
        y1 = torch.empty(M, device=dev, dtype=torch.float16)

        def one(i):
            lib.check(L.rwkv_mm8_one_f16(N, M, x1.data_ptr(), w[i % ncopy].data_ptr(), 1, N, mx.data_ptr(), rx.data_ptr(),
                                         my.data_ptr(), ry.data_ptr(), y1.data_ptr(), lib.RWKV_DT_F16, st), "rwkv_mm8_one_f16")
        T = 1024
        xs = torch.randn(T, N, device=dev).half()
        ys = torch.empty(T, M, device=dev, dtype=torch.float16)
        nbytes = L.rwkv_mm8_seq_workspace(T, N)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)

        def seq(i):
            lib.check(L.rwkv_mm8_seq_f16(T, N, M, xs.data_ptr(), N, w[i % ncopy].data_ptr(), 1, N, mx.data_ptr(), rx.data_ptr(),
                                         my.data_ptr(), ry.data_ptr(), ys.data_ptr(), M, ws.data_ptr(), nbytes, st),
                      "rwkv_mm8_seq_f16")
        for name, fn, n in (("mm8_one", one, reps), ("mm8_seq", seq, max(4, reps // 2))):
            for i in range(3):
                fn(i)
            k = [0]

            def warm():
                k[0] += 1
                fn(k[0])
            spin_up(warm, min(SPINUP_S, 0.3), sync_every=64)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(n):
                fn(i)
            e1.record()
            torch.cuda.synchronize()
            t = e0.elapsed_time(e1) * 1e-3 / n
            if name == "mm8_one":
                out[f"mm8_one [{N}] x [{N} x {M}]"] = {"us": t * 1e6, "GBps": N * M / t / 1e9, "frac_of_hbm_peak": N * M / t / HBM_PEAK}
            else:
                out[f"mm8_seq [{T} x {N}] x [{N} x {M}]"] = {"us": t * 1e6, "TFLOPs": 2.0 * T * N * M / t / 1e12,
                                                           "frac_of_mfma_peak": 2.0 * T * N * M / t / MFMA_F16_PEAK}
        del w
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--spinup", type=float, default=1.0,
                    help="seconds of the same work run untimed right before every timed region, on top of --warmup: "
                         "the shader clock takes tens of milliseconds of continuous load to rise from its idle level "
                         "(1.4 GHz in a cold 4 ms burst, 1.8 GHz sustained, measured with the cycle counter)")
    ap.add_argument("--shape", default="v4-7b")
    ap.add_argument("--strategy", default="cuda fp16i8")
    ap.add_argument("--prefill", type=int, default=1024)
    ap.add_argument("--chunk", type=int, default=0, help="prefill in calls of this many tokens (0: one call)")
    ap.add_argument("--layers", type=int, default=None, help="debug: fewer layers (result is then not the headline)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--select", choices=["greedy", "torch"], default="greedy",
                    help="next token on the device by rwkv_greedy_token (one launch) or by torch's argmax + conversion")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run five plain 1 GiB device copies (a kernel of known HBM traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; the path has no multi-GPU mode (--gpus must be 1)",
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from chatrwkv_amd import synth
    from chatrwkv_amd.model import RWKV

    version, L, C, F, V = synth.SHAPES[args.shape]
    if args.layers:
        L = args.layers
    dev = "cuda:0"
    torch.cuda.set_device(0)
    u8 = args.strategy.endswith("i8")
    if version == 7:
        # RWKV-7 runs unquantised (the reference offers fp16 / bf16 / fp32 only)
        from chatrwkv_amd.model_v7 import RWKV_x070
        ck = synth.make_checkpoint_v7(n_layer=L, n_embd=C, n_ffn=F, vocab=V, seed=2, device=dev)
        model = RWKV_x070(ck, args.strategy)
        wbytes = 2 * (L * (4 * C * C + 2 * C * F + 2 * C * sum(synth.v7_lora_dims(C))) + C * V)
    else:
        ck = synth.make_checkpoint(version=version, n_layer=L, n_embd=C, n_ffn=F, vocab=V, seed=2, device=dev)
        model = RWKV(ck, args.strategy, verbose=False)
        wbytes = u8_weight_bytes(L, C, F, V, version) * (1 if u8 else 2)
    del ck
    torch.cuda.empty_cache()

    # ---- prefill: one call over `prefill` tokens (median of 5 calls queued back to back, after the spin-up)
    ptoks = synth.random_tokens(args.prefill, V, seed=2)
    chunk = args.chunk if args.chunk > 0 else args.prefill

    def prefill():
        out, state = None, None
        for i in range(0, len(ptoks), chunk):
            out, state = model.forward(ptoks[i:i + chunk], state)
        return out, state

    global SPINUP_S
    SPINUP_S = args.spinup
    prefill()
    spin_up(prefill, args.spinup)
    pt, evs = [], []
    for _ in range(5):      # queued back to back: no idle gap between the calls
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        out, state = prefill()
        e1.record()
        evs.append((e0, e1))
    torch.cuda.synchronize()
    pt = [e0.elapsed_time(e1) * 1e-3 for e0, e1 in evs]
    t_prefill = float(np.median(pt))
    prefill_flops = 2.0 * args.prefill * (wbytes / (1 if u8 else 2) - C * V) + 2.0 * C * V

    # ---- decode: W warm-up + K timed greedy steps, token stays on the device
    if args.select == "greedy":
        from chatrwkv_amd.sampling import greedy_token as pick
    else:
        def pick(logits, into=None):
            return logits.argmax().reshape(1).to(torch.int32)
    tok = pick(out, model.token_slot)   # the id is written where the one-token step reads it: no copy per step
    def one_step():
        nonlocal out, state, tok
        out, state = model.forward(tok, state)
        tok = pick(out, tok)
    for _ in range(args.warmup):
        one_step()
    n_spin = spin_up(one_step, args.spinup, sync_every=64)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out, state = model.forward(tok, state)
        tok = pick(out, tok)
    torch.cuda.synchronize()
    t_dev = time.perf_counter() - t0

    # the same K steps with the token fetched to the host every step (what a sampling caller does)
    t0 = time.perf_counter()
    nxt = int(tok)
    for _ in range(args.steps):
        out, state = model.forward([nxt], state)
        nxt = int(out.argmax())
    torch.cuda.synchronize()
    t_host = time.perf_counter() - t0

    # ---- per-kernel durations: each decode phase launched back to back over all layers (every
    # layer streams its own weights, so nothing is served from cache) between two HIP events
    torch.cuda.synchronize()
    tok_s = args.steps / t_dev
    if version == 4:
        names = ["att_kvr_wkv", "att_output", "ffn_rk", "ffn_value", "head"]
        scale = 1 if u8 else 2
        kbytes = {"att_kvr_wkv": 3 * C * C * scale, "att_output": C * C * scale, "ffn_rk": (C * C + C * F) * scale,
                  "ffn_value": C * F * scale, "head": C * V * scale}
        kms = {n: model.time_phase(j, reps=(8 if n != "head" else 64)) for j, n in enumerate(names)}
        ktot = {n: kms[n] * (L if n != "head" else 1) for n in kms}
        dom = max(ktot, key=ktot.get)
        kernels = {n: {"ms": round(kms[n], 5), "bytes": kbytes[n], "GBps": round(kbytes[n] / (kms[n] * 1e-3) / 1e9, 1)}
                   for n in kms}
        kname = {"att_kvr_wkv": "att_kernel", "att_output": "vec_kernel", "ffn_rk": "lnmix_kernel",
                 "ffn_value": "vec_kernel", "head": "lnmix_kernel"}[dom] + f" ({dom})"
        roof = {"bound": "hbm", "kernel": kname, "achieved": kbytes[dom] / (kms[dom] * 1e-3) / 1e9,
                "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": kbytes[dom] / (kms[dom] * 1e-3) / HBM_PEAK,
                "traffic": MEASURED_TRAFFIC.get((args.shape, args.strategy, L, dom)),
                "traffic_source": TRAFFIC_SOURCE if (args.shape, args.strategy, L, dom) in MEASURED_TRAFFIC else None,
                "bytes_per_launch": kbytes[dom], "ms_per_launch": kms[dom]}
    else:
        # RWKV-5/6 one-token steps are a chain of the same streaming GEMV launches with no per-phase timing
        # entry; the roofline figure is then the whole step: uint8 matrix bytes per token over the step time
        kernels = None
        roof = {"bound": "hbm", "kernel": "whole one-token step (vec_kernel chain)", "achieved": wbytes * tok_s / 1e9,
                "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": wbytes * tok_s / HBM_PEAK, "traffic": None,
                "bytes_per_launch": wbytes, "ms_per_launch": 1e3 / tok_s}

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    res = {
        "metric": "7B fp16i8 decode tok/s (% HBM peak) + prefill tok/s, 1 MI355X" if args.shape == "v4-7b" and u8 else
                  f"{args.shape} '{args.strategy}' decode tok/s (% HBM peak) + prefill tok/s, 1 MI355X",
        "value": tok_s, "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "spinup_s": args.spinup, "spinup_steps": n_spin,
        "ms_per_step": 1e3 * t_dev / args.steps, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u8 weights, fp16 activations, fp32 accumulate" if u8 else "fp16",
        "data": "synthetic (random-init weights, random tokens)",
        "config": {"workload": f"RWKV-{int(version)} {args.shape} ({L} layers, n_embd {C}, ffn {F}, vocab {V}) '{args.strategy}', "
                               f"batch 1: prefill {args.prefill} tokens in {'one call' if chunk >= args.prefill else f'calls of {chunk}'}, "
                               f"then greedy decode" + (" (BASELINE.json configs[2])" if args.shape == "v4-7b" else ""),
                   "strategy": args.strategy, "prefill_tokens": args.prefill,
                   "next_token": "rwkv_greedy_token (argmax of the logits, one launch, id stays on the device)"
                                 if args.select == "greedy" else "torch argmax + conversion to int32 on the device"},
        "roofline": roof,
        "decode_hbm": {"weight_bytes_per_token": wbytes, "achieved_GBps": wbytes * tok_s / 1e9,
                       "frac_of_peak": wbytes * tok_s / HBM_PEAK},
        "decode_tok_s_host_sync": args.steps / t_host,
        "decode_kernels": kernels,
        "prefill": {"tokens": args.prefill, "tok_s": args.prefill / t_prefill, "ms": 1e3 * t_prefill,
                    "flops": prefill_flops, "TFLOPs": prefill_flops / t_prefill / 1e12,
                    "frac_of_mfma_peak": prefill_flops / t_prefill / MFMA_F16_PEAK},
        "prefill_roofline": gemm_roofline(min(chunk, args.prefill), C, F, u8),
    }
    if args.shape == "v4-7b" and u8:
        res["isolated_mm8_op"] = isolated_mm8()
    if not args.no_cpu and version != 7:
        # the CPU baseline proper: configs[0] in full; beside it one layer + head of the benchmarked shape
        res["cpu_baseline"] = cpu_baseline_cfg0()
        res["cpu_baseline_layer_sample"] = cpu_baseline(args.shape, budget_s=12.0)
    else:
        res["cpu_baseline"] = None
    print(json.dumps(res))


if __name__ == "__main__":
    main()
