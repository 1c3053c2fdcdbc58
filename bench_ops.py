#!/usr/bin/env python3
"""Operator sweep on one MI355X: the kernel families of the token loop measured one by one.

  * measured ceilings: int8 matrix-core rate (register-only MFMA loop) and HBM read rate (2 GiB scan),
    printed next to the published peaks every fraction below divides by (8 TB/s, 5 POP/s);
  * GEMV (one activation row) over M x K in {4096x4096, 11008x4096, 4096x11008, 32000x4096} x
    {Q4_0, Q8_0, Q4_K, Q6_K} weights x Q8_0 activations: bytes = M*K*bytes-per-weight, against HBM;
  * GEMM, the same weights x {16, 128, 512} activation rows: 2*T*M*K operations against the int8 MFMA
    peak (T = 16 is still bandwidth-bound: its HBM fraction is printed too);
  * decode attention, 32 heads x 128, f16 K cache [token][head][128] and transposed V cache, at
    n_kv in {512, 4096}: scores + softmax/PV kernels (bytes = 2*n_kv*4096*2) and the fused attention
    launch of a layer (which also reads wq, wk, wv).

Every timed loop walks over enough distinct copies of its operands (>= 600 MB) that nothing is served
from a cache the token loop would not have.  Activations are seeded N(0,1) quantized on the device;
Q4_0 / Q8_0 weights are seeded N(0, 0.02) quantized with the GGUF rule, K-quant weights are random
well-formed blocks.  Prints a markdown report; --json adds one JSON line per measurement.
"""
import argparse
import ctypes as C
import json
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

HBM_PEAK = 8.0e12
INT8_PEAK = 5.0e15
SHAPES = [(4096, 4096), (11008, 4096), (4096, 11008), (32000, 4096)]
TYPE_NAMES = {2: "Q4_0", 8: "Q8_0", 12: "Q4_K", 14: "Q6_K"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--json", action="store_true")
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--skip", default="", help="comma list of: peaks, gemv, gemm, prompt_attention, exact_prompt, attention")
    args = ap.parse_args()
    skip = set(args.skip.split(",")) if args.skip else set()

    from spy_amd import _lib as H, model as M
    H.init(0)
    L = H.load()
    recs = []

    def emit(rec):
        recs.append(rec)
        if args.json:
            print(json.dumps(rec), flush=True)

    e0, e1 = C.c_void_p(), C.c_void_p()
    H.check(L.spy_hip_event_create(C.byref(e0)), "event")
    H.check(L.spy_hip_event_create(C.byref(e1)), "event")

    # Kernels of a few microseconds cannot be timed by launching them one by one from Python: the host
    # needs longer per launch than the GPU per kernel.  A blocker (fills of a 1 GiB buffer) keeps the GPU
    # busy while the timed launches and both events are enqueued behind it, so that they then run back to
    # back; the blocker is sized from the measured host cost per launch.
    blocker = H.DeviceBuffer(1 << 30)
    H.check(L.spy_hip_fill_u8(blocker.ptr, 0, blocker.nbytes, None), "fill")
    H.sync()
    H.check(L.spy_hip_event_record(e0, None), "record")
    for _ in range(4):
        H.check(L.spy_hip_fill_u8(blocker.ptr, 0, blocker.nbytes, None), "fill")
    H.check(L.spy_hip_event_record(e1, None), "record")
    ms = C.c_float()
    H.check(L.spy_hip_event_elapsed_ms(e0, e1, C.byref(ms)), "elapsed")
    fill_us = ms.value * 1000.0 / 4

    def time_us(fn, n_launch):
        """fn() enqueues n_launch kernels (one per operand copy); returns GPU microseconds per launch."""
        import time
        fn()                                       # warm-up pass over all copies
        H.sync()
        t0 = time.perf_counter()
        fn()
        host_us = (time.perf_counter() - t0) * 1e6 / n_launch
        H.sync()
        reps = max(1, min(args.reps, 600 // n_launch))
        n_fill = int(host_us * 1.5 * reps * n_launch / fill_us) + 2
        for _ in range(n_fill):
            H.check(L.spy_hip_fill_u8(blocker.ptr, 0, blocker.nbytes, None), "fill")
        H.check(L.spy_hip_event_record(e0, None), "record")
        for _ in range(reps):
            fn()
        H.check(L.spy_hip_event_record(e1, None), "record")
        ms = C.c_float()
        H.check(L.spy_hip_event_elapsed_ms(e0, e1, C.byref(ms)), "elapsed")
        return ms.value * 1000.0 / (reps * n_launch)

    info = H.device_info()
    print("# Operator sweep — %s, %d CUs\n" % (info["name"].strip(), info["num_cu"]), flush=True)

    if "peaks" not in skip:
        tops, gbps = C.c_float(), C.c_float()
        H.check(L.spy_hip_measure_mfma_i8(None, 20000, C.byref(tops)), "spy_hip_measure_mfma_i8")
        sc = [C.c_float(), C.c_float()]
        for mode in (0, 1):
            H.check(L.spy_hip_measure_mfma_i8_scaled(None, 20000, mode, C.byref(sc[mode])), "spy_hip_measure_mfma_i8_scaled")
        buf = H.DeviceBuffer(2 << 30)
        H.check(L.spy_hip_fill_u8(buf.ptr, 1, buf.nbytes, None), "fill")
        H.check(L.spy_hip_measure_hbm_read(None, buf.ptr, buf.nbytes, 10, C.byref(gbps)), "spy_hip_measure_hbm_read")
        buf.free()
        print("## Measured ceilings\n")
        print("| what | measured | published peak used as denominator | measured / published |")
        print("|---|---|---|---|")
        print("| int8 MFMA, register operands only (`v_mfma_i32_32x32x32_i8`) | %.0f TOP/s | 5000 TOP/s | %.2f |" % (tops.value, tops.value * 1e12 / INT8_PEAK))
        print("| the same MFMA + fp16 scale outer product + conversion and fma per output (block-scaled GEMM inner loop, registers only) | %.0f TOP/s | 5000 TOP/s | %.2f |" % (sc[0].value, sc[0].value * 1e12 / INT8_PEAK))
        print("| ... with the accumulator biased by 0x4B400000 and a subtraction in place of the conversion (what `spy_hip_gemm_q8_0act` runs) | %.0f TOP/s | 5000 TOP/s | %.2f |" % (sc[1].value, sc[1].value * 1e12 / INT8_PEAK))
        print("| HBM read, 2 GiB scan | %.0f GB/s | 8000 GB/s | %.2f |\n" % (gbps.value, gbps.value * 1e9 / HBM_PEAK), flush=True)
        emit({"op": "peak_mfma_i8", "tops": tops.value})
        emit({"op": "peak_mfma_i8_scaled_cvt", "tops": sc[0].value})
        emit({"op": "peak_mfma_i8_scaled_biased", "tops": sc[1].value})
        emit({"op": "peak_hbm_read", "gbps": gbps.value})

    def weights(wt, M_, K):
        n = M_ * K
        return M.synth_tensor(wt, 7, "sweep.%d.%d.%d" % (wt, M_, K), n)

    def activations(T, K):
        x = np.random.default_rng(T * 131 + K).standard_normal((T, K)).astype(np.float32)
        dx = H.DeviceBuffer.from_numpy(x)
        dq = H.DeviceBuffer(T * (K // 32) * 34)
        H.check(L.spy_hip_quantize_q8_0(None, dx.ptr, K, dq.ptr, T, K), "spy_hip_quantize_q8_0")
        H.sync()
        dx.free()
        return dq

    if "gemv" not in skip or "gemm" not in skip:
        rows_gemv, rows_gemm = [], []
        for wt in (H.Q4_0, H.Q8_0, H.Q4_K, H.Q6_K):
            for (M_, K) in SHAPES:
                w = weights(wt, M_, K)
                ncopy = max(2, -(-600_000_000 // w.nbytes))
                copies = [H.DeviceBuffer.from_numpy(w) for _ in range(ncopy)]
                if "gemv" not in skip:
                    xq = activations(1, K)
                    out = H.DeviceBuffer(M_ * 4)

                    def run():
                        for c in copies:
                            H.check(L.spy_hip_gemv_q8_0act(None, wt, c.ptr, xq.ptr, out.ptr, None, M_, K, 1, M_), "spy_hip_gemv_q8_0act")
                    us = time_us(run, ncopy)
                    rows_gemv.append((TYPE_NAMES[wt], M_, K, w.nbytes, us))
                    emit({"op": "gemv", "type": TYPE_NAMES[wt], "M": M_, "K": K, "bytes": int(w.nbytes), "us": us,
                          "gbps": w.nbytes / us / 1e3, "hbm_frac": w.nbytes / (us * 1e-6) / HBM_PEAK})
                    xq.free(); out.free()
                if "gemm" not in skip:
                    for T in (16, 128, 512):
                        xq = activations(T, K)
                        out = H.DeviceBuffer(T * M_ * 4)

                        def run():
                            for c in copies:
                                H.check(L.spy_hip_gemm_q8_0act(None, wt, c.ptr, xq.ptr, out.ptr, M_, K, T, M_), "spy_hip_gemm_q8_0act")
                        us = time_us(run, ncopy)
                        rows_gemm.append((TYPE_NAMES[wt], M_, K, T, w.nbytes, us))
                        emit({"op": "gemm", "type": TYPE_NAMES[wt], "M": M_, "K": K, "T": T, "us": us, "tops": 2.0 * T * M_ * K / us / 1e6,
                              "mfma_frac": 2.0 * T * M_ * K / (us * 1e-6) / INT8_PEAK, "hbm_frac": w.nbytes / (us * 1e-6) / HBM_PEAK})
                        xq.free(); out.free()
                for c in copies:
                    c.free()
        if rows_gemv:
            print("## GEMV, one activation row (`spy_hip_gemv_q8_0act`): against HBM\n")
            print("| weights | M x K | bytes | µs at 8 TB/s | measured µs | GB/s | of 8 TB/s |")
            print("|---|---|---|---|---|---|---|")
            for (tn, M_, K, nb, us) in rows_gemv:
                print("| %s | %d x %d | %d | %.2f | %.2f | %.0f | %.2f |" % (tn, M_, K, nb, nb / HBM_PEAK * 1e6, us, nb / us / 1e3, nb / (us * 1e-6) / HBM_PEAK))
            print(flush=True)
        if rows_gemm:
            print("## GEMM, T activation rows (`spy_hip_gemm_q8_0act`): against the int8 MFMA peak\n")
            print("| weights | M x K | T | measured µs | TOP/s | of 5 POP/s | weight bytes / time, of 8 TB/s |")
            print("|---|---|---|---|---|---|---|")
            for (tn, M_, K, T, nb, us) in rows_gemm:
                ops = 2.0 * T * M_ * K
                print("| %s | %d x %d | %d | %.1f | %.0f | %.3f | %.2f |" % (tn, M_, K, T, us, ops / us / 1e6, ops / (us * 1e-6) / INT8_PEAK, nb / (us * 1e-6) / HBM_PEAK))
            print(flush=True)

    if "prompt_attention" not in skip:
        print("## Prompt attention, 32 heads x 128, f16 KV, one chunk of 2048 queries (`spy_hip_prompt_attention`): against the fp16 MFMA peak\n")
        print("| cached before | queries | measured µs | useful TFLOP/s (causal q.K and P.V^T once) | of 2.5 PFLOP/s |")
        print("|---|---|---|---|---|")
        Hh, hd, T, n_ctx = 32, 128, 2048, 4096
        rng = np.random.default_rng(5)
        dq = H.DeviceBuffer.from_numpy(rng.standard_normal((Hh, T, hd)).astype(np.float16))
        dk = H.DeviceBuffer.from_numpy(rng.standard_normal((n_ctx, Hh * hd)).astype(np.float16))
        dv = H.DeviceBuffer.from_numpy(rng.standard_normal((Hh * hd, n_ctx)).astype(np.float16))
        do = H.DeviceBuffer(T * Hh * hd * 4)
        tot = 0.0
        for past in (0, 2048):
            def run():
                H.check(L.spy_hip_prompt_attention(None, dq.ptr, dk.ptr, dv.ptr, do.ptr, T, Hh, hd, past, n_ctx, 1.0 / np.sqrt(hd)), "spy_hip_prompt_attention")
            us = time_us(run, 1)
            pairs = T * past + T * (T + 1) / 2                       # (query, visible position) pairs per head
            flops = 2.0 * 2.0 * hd * pairs * Hh
            tot += us
            print("| %d | %d | %.1f | %.0f | %.3f |" % (past, T, us, flops / us / 1e6, flops / (us * 1e-6) / 2.5e15), flush=True)
            emit({"op": "prompt_attention", "past": past, "T": T, "us": us, "tflops": flops / us / 1e6})
        print("\nmean of the two chunks of a 4096-token prompt: %.1f µs per layer and chunk\n" % (tot / 2), flush=True)
        for b in (dq, dk, dv, do):
            b.free()

    if "exact_prompt" not in skip:
        # the prompt kernels of summation order 1: tiled exact MatMul (`spy_hip_op_matmul` with the exact-order switch on, activations
        # quantized inside the call) and the three causal attention kernels behind `spy_hip_prompt_attention_exact`
        print("## Prompt kernels in the host backend's summation order (order 1): tiled exact MatMul and causal exact attention, 2048 activation rows\n")
        print("| weights | M x K | T | measured µs (Q8_0 quantization of the activations included) | TMAC/s |")
        print("|---|---|---|---|---|")
        prev = L.spy_hip_set_exact_order(1)
        T = 2048
        for wt in (H.Q4_0, H.Q8_0, H.Q4_K, H.Q6_K):
            for (M_, K) in ((4096, 4096), (11008, 4096), (4096, 11008)):
                w = weights(wt, M_, K)
                dw = H.DeviceBuffer.from_numpy(w)
                dx = H.DeviceBuffer.from_numpy(np.random.default_rng(M_ + K).standard_normal((T, K)).astype(np.float32))
                dd = H.DeviceBuffer(T * M_ * 4)
                tw, tx, td = H.tensor(dw, wt, [K, M_]), H.tensor(dx, H.F32, [K, T]), H.tensor(dd, H.F32, [M_, T])
                need = L.spy_hip_op_matmul_scratch_size(C.byref(tw), C.byref(tx))
                scr = H.DeviceBuffer(need)

                def run():
                    H.check(L.spy_hip_op_matmul(None, C.byref(tw), C.byref(tx), C.byref(td), scr.ptr, need), "spy_hip_op_matmul")
                us = time_us(run, 1)
                print("| %s | %d x %d | %d | %.1f | %.1f |" % (TYPE_NAMES[wt], M_, K, T, us, T * M_ * K / us / 1e6), flush=True)
                emit({"op": "exact_matmul", "wtype": TYPE_NAMES[wt], "M": M_, "K": K, "T": T, "us": us, "tmacs": T * M_ * K / us / 1e6})
                for b in (dw, dx, dd, scr):
                    b.free()
        L.spy_hip_set_exact_order(prev)
        print()
        print("| cached before | queries | measured µs (scores + softmax + product with V^T) | fp32 fmas per second, T (256 per pair of a query and a visible position) |")
        print("|---|---|---|---|")
        Hh, hd, n_ctx = 32, 128, 4096
        rng = np.random.default_rng(6)
        dq = H.DeviceBuffer.from_numpy(rng.standard_normal((T, Hh * hd)).astype(np.float32))
        dk = H.DeviceBuffer.from_numpy(rng.standard_normal((n_ctx, Hh * hd)).astype(np.float16))
        dv = H.DeviceBuffer.from_numpy(rng.standard_normal((Hh * hd, n_ctx)).astype(np.float16))
        do = H.DeviceBuffer(T * Hh * hd * 4)
        for past in (0, 2048):
            need = L.spy_hip_prompt_attention_exact_scratch_size(T, Hh, past)
            scr = H.DeviceBuffer(need)

            def run():
                H.check(L.spy_hip_prompt_attention_exact(None, dq.ptr, dk.ptr, dv.ptr, do.ptr, T, Hh, hd, past, n_ctx, past + T, 1.0 / np.sqrt(hd), scr.ptr, need),
                        "spy_hip_prompt_attention_exact")
            us = time_us(run, 3)
            pairs = (T * past + T * (T + 1) / 2) * Hh
            print("| %d | %d | %.1f | %.1f |" % (past, T, us * 3, pairs * 256 / (us * 3) / 1e6), flush=True)
            emit({"op": "prompt_attention_exact", "past": past, "T": T, "us": us * 3})
            scr.free()
        print(flush=True)
        for b in (dq, dk, dv, do):
            b.free()

    if "attention" not in skip:
        print("## Decode attention, 32 heads x 128, f16 KV (kernels of the single-token pass, 8 layers walked in turn)\n")
        print("| n_kv | kernels | bytes per launch | µs at 8 TB/s | measured µs | GB/s | of 8 TB/s |")
        print("|---|---|---|---|---|---|---|")
        cfg = M.Config.llama2_7b(n_ctx=4352, wtype=H.Q4_0)
        cfg.n_layer = 8
        tensors = M.synth_model(cfg, seed=11)
        for mode in ("own_split", "own_fused", "host_order"):
            split = mode == "own_split"
            if split:
                os.environ["SPY_HIP_ATTN_SPLIT"] = "1"
            else:
                os.environ.pop("SPY_HIP_ATTN_SPLIT", None)
            eng = M.Engine(cfg, tensors, order=1 if mode == "host_order" else 0)
            for n_kv in (512, 4096):
                eng.forward(np.array([1], np.int32), n_kv - 1, want_logits=False)       # leaves position n_kv - 1
                kv = 2 * n_kv * cfg.n_embd * 2
                if mode == "host_order":
                    s_us, p_us = eng.kernel_time_us("scores", args.reps), eng.kernel_time_us("pv", args.reps)
                    us, nb, label = s_us + p_us, kv, "host summation order: `xattn_scores_kernel` %.2f + `xattn_pv_kernel` %.2f" % (s_us, p_us)
                elif split:
                    s_us, p_us = eng.kernel_time_us("scores", args.reps), eng.kernel_time_us("pv", args.reps)
                    us, nb, label = s_us + p_us, kv, "`attn_scores_kernel` %.2f + `attn_pv_kernel` %.2f" % (s_us, p_us)
                elif eng.fuses_attention():
                    us = eng.kernel_time_us("qkv", args.reps)
                    nb, label = kv + 3 * H.row_size(H.Q4_0, cfg.n_embd * cfg.n_embd), "`attn_layer_kernel` (norm, wq/wk/wv Q4_0, RoPE, cache write, scores, softmax, PV)"
                else:
                    continue
                print("| %d | %s | %d | %.2f | %.2f | %.0f | %.2f |" % (n_kv, label, nb, nb / HBM_PEAK * 1e6, us, nb / us / 1e3, nb / (us * 1e-6) / HBM_PEAK), flush=True)
                emit({"op": "attention_" + mode, "n_kv": n_kv, "bytes": nb, "us": us, "hbm_frac": nb / (us * 1e-6) / HBM_PEAK})
            eng.close()
        print(flush=True)


if __name__ == "__main__":
    main()
