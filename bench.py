#!/usr/bin/env python3
"""Headline benchmark: single-sequence greedy decode of a LLaMA-2-7B shaped Q4_0 model with the
f16 KV cache filled to 4096 tokens, on one MI355X.

A "step" is one single-token forward pass (all 32 layers + output head + greedy sampling) at
n_kv = 4096 + step; weights and KV cache are resident in HBM before the timed region starts.
Prints ONE JSON line (see the keys below).  The CPU baseline is the oracle (a port of the reference's
host backend path) timed on this machine's cores on a bounded sample of the same workload.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12          # MI355X HBM3E, bytes/s
INT8_PEAK = 5.0e15         # MI355X dense int8 MFMA, op/s


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--ctx-fill", type=int, default=4096, help="tokens in the KV cache before the first timed step")
    ap.add_argument("--prefill", choices=["real", "synthetic"], default="real",
                    help="real: run the prompt through the model; synthetic: fill the caches with random fp16 (quick runs)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-steps", type=int, default=8)
    ap.add_argument("--cpu-threads", type=int, default=8, help="threads of the CPU baseline (the reference's configurations name -t 8)")
    ap.add_argument("--layers", type=int, default=32, help="debug only: fewer layers (result is then not the headline config)")
    ap.add_argument("--model", choices=["q4_0", "q8_0", "q4_k_m"], default="q4_0",
                    help="q4_0: the headline workload; q8_0 / q4_k_m (Q4_K with Q6_K attn_v, ffn_down and head): the other 7B configurations")
    ap.add_argument("--head", choices=["q6_k", "body"], default="q6_k",
                    help="--model q4_0 only: output head in Q6_K (the named configuration; default) or in the body's Q4_0 (the variant Spy's CPU backend can run)")
    ap.add_argument("--via-gguf", metavar="PATH", default=None,
                    help="write the synthetic model to PATH as a GGUF file and run the model loaded from it (file -> HBM times are reported)")
    ap.add_argument("--no-gemm", action="store_true", help="skip the timing of the prompt's quantized GEMM")
    ap.add_argument("--no-graph", action="store_true", help="launch the kernels of every pass one by one instead of replaying a HIP graph (for profilers)")
    ap.add_argument("--order", type=int, choices=[0, 1], default=1,
                    help="with --only-order: the one summation order to time (1 = the host backend's, 0 = this backend's own); by default both are timed and 1 is the headline")
    ap.add_argument("--only-order", action="store_true", help="time one summation order only (profiling runs)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch a plain copy kernel over 256 MiB three times (a known-size dispatch to scale profiler byte counters by)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the token loop on ONE GPU (no sharding, no collectives); --gpus %d is not supported" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    from spy_amd import _lib as H
    from spy_amd import model as M

    H.init(0)
    info = H.device_info()
    log("device:", info)
    steps, warmup, fill = args.steps, args.warmup, args.ctx_fill
    n_ctx = (fill + warmup + steps + 8 + 63) // 64 * 64
    if args.model == "q4_0":
        cfg = M.Config.llama2_7b(n_ctx=n_ctx, wtype=H.Q4_0, t_out=H.Q4_0 if args.head == "body" else H.Q6_K)
    elif args.model == "q8_0":
        cfg = M.Config.llama2_7b(n_ctx=n_ctx, wtype=H.Q8_0)
    else:
        cfg = M.Config.llama2_7b(n_ctx=n_ctx, wtype=H.Q4_K, t_out=H.Q6_K, tensor_types={"attn_v": H.Q6_K, "ffn_down": H.Q6_K})
    cfg.n_layer = args.layers
    t0 = time.time()
    tensors = M.synth_model(cfg, seed=1234, outlier_every=1000 if args.model == "q4_k_m" else 0)   # the Q4_K_M configuration: 0.1 % of the weights x 20
    log("synthetic model: %.1f s, %.2f GB of weights streamed per token" % (time.time() - t0, cfg.weight_bytes() / 1e9))
    load_info, loaded = None, None
    if args.via_gguf:
        from spy_amd import gguf as G
        t0 = time.time()
        G.write_llama(args.via_gguf, cfg, tensors)
        t_write = time.time() - t0
        loaded = G.GGUFModel(args.via_gguf, n_ctx=n_ctx)
        eng = loaded.engine
        load_info = {"file_bytes": os.path.getsize(args.via_gguf), "parse_ms": round(loaded.parse_ms, 2), "upload_ms": round(loaded.upload_ms, 1),
                     "create_ms": round(loaded.create_ms, 1), "upload_GBps": round(loaded.weight_bytes / loaded.upload_ms / 1e6, 2)}
        log("GGUF: wrote %.2f GB in %.1f s; parse %.1f ms, upload to HBM %.0f ms (%.1f GB/s from the page cache), token loop set-up %.0f ms"
            % (load_info["file_bytes"] / 1e9, t_write, loaded.parse_ms, loaded.upload_ms, load_info["upload_GBps"], loaded.create_ms))
    else:
        eng = M.Engine(cfg, tensors)
    rng = np.random.default_rng(4096)
    prompt = rng.integers(0, cfg.n_vocab, fill).astype(np.int32)

    # The prompt pass, output head on the last token only.  A model in order 1 runs it in the host backend's order as well (tiled exact
    # kernels, vector units), a model in order 0 on the matrix cores; each order's single-token passes below start from its own prompt pass.
    def prefill(order):
        eng.set_order(order)
        t0 = time.time()
        if args.prefill == "real":
            first = int(np.argmax(eng.forward_last(prompt, 0)))
        else:
            for il in range(cfg.n_layer):
                eng.write_buffer("k_cache", il, (rng.standard_normal(fill * cfg.n_embd) * 1.3).astype(np.float16).view(np.uint16))
                v = np.zeros((cfg.n_embd, cfg.n_ctx), np.float16)
                v[:, :fill] = (rng.standard_normal((cfg.n_embd, fill)) * 1.3).astype(np.float16)
                eng.write_buffer("v_cache", il, v.view(np.uint16))
            first = int(prompt[-1])
        H.sync()
        dt = time.time() - t0
        log("order %d prefill (%s) of %d tokens: %.2f s" % (order, args.prefill, fill, dt))
        return first, dt
    if args.calibrate:
        n = 64 << 20
        src, dst = H.DeviceBuffer(n * 4), H.DeviceBuffer(n * 4)
        src.fill(0)
        ts, td = H.tensor(src, H.F32, [n]), H.tensor(dst, H.F32, [n])
        for _ in range(3):
            H.check(H.load().spy_hip_op_dup(None, C.byref(ts), C.byref(td)), "spy_hip_op_dup")
        H.sync()
        log("calibration: dup_kernel over %d bytes read + %d bytes written, 3 launches" % (n * 4, n * 4))

    # Two summation orders of the single-token pass are timed on the same cache, from the same position:
    #   order 1 (headline): the host backend's order -- the path whose greedy tokens and logits equal the CPU oracle's bit for bit;
    #   order 0: this backend's own lane-parallel order (per-operator results equal to ~1e-7, greedy tokens of near-tied logits may differ).
    # Each: warm-up passes (the first also captures the HIP graphs), then exactly `steps` timed passes.
    d, F, V = cfg.n_embd, cfg.n_ff, cfg.n_vocab
    kv_bytes = 2 * cfg.n_embd * 2 * cfg.n_layer           # K and V, fp16, per cached token
    tt = lambda n: cfg.tensor_types.get(n, cfg.wtype)
    rs = H.row_size
    tn = {H.Q4_0: "Q4_0", H.Q8_0: "Q8_0", H.Q4_K: "Q4_K", H.Q6_K: "Q6_K"}
    traffic_db = {}
    tpath = os.path.join(ROOT, "profiles", "decode_hbm_traffic.json")      # FETCH_SIZE / WRITE_SIZE per dispatch, scaled by a copy kernel (see the file)
    if os.path.exists(tpath):
        with open(tpath) as f:
            traffic_db = json.load(f)

    prefill_s, firsts = {}, {}

    def run_order(order):
        first, prefill_s[order] = prefill(order)
        firsts[order] = first
        pos = fill
        toks = eng.decode_greedy(first, pos, warmup, use_graph=not args.no_graph)
        pos += warmup
        eng.timing()
        H.sync()
        t0 = time.perf_counter()
        toks = eng.decode_greedy(int(toks[-1]), pos, steps, use_graph=not args.no_graph)
        H.sync()
        wall = time.perf_counter() - t0
        ev_ms, n_timed = eng.timing()
        assert n_timed == steps
        n_kv_mid = pos + steps / 2.0
        bytes_per_token = cfg.weight_bytes() + kv_bytes * n_kv_mid
        frac = bytes_per_token / (wall / steps) / HBM_PEAK
        log("order %d decode: %.3f ms/step wall, %.3f ms/step by HIP events, %.1f tok/s, %.2f GB/token -> %.1f%% of 8 TB/s"
            % (order, wall * 1e3 / steps, ev_ms, steps / wall, bytes_per_token / 1e9, 100 * frac))
        # per-kernel times: HIP events around repeated launches of each kernel of a layer, on the stream they run on, at the last position
        per_kernel = {}
        for name in ("qkv", "scores", "pv", "wo", "gate_up", "down", "head"):
            per_kernel[name] = eng.kernel_time_us(name, reps=4)
        n_kv_end = pos + steps
        alg = {"qkv": d * (rs(tt("attn_q"), d) + rs(tt("attn_k"), d) + rs(tt("attn_v"), d)), "wo": d * rs(tt("attn_output"), d),
               "gate_up": F * (rs(tt("ffn_gate"), d) + rs(tt("ffn_up"), d)), "down": d * rs(tt("ffn_down"), F),
               "head": V * rs(cfg.t_out, d), "scores": n_kv_end * d * 2, "pv": n_kv_end * d * 2}
        if eng.fuses_attention():           # qkv, scores and softmax + KQV are one launch, timed under "qkv"
            per_kernel["attention"] = per_kernel.pop("qkv")
            alg["attention"] = alg["qkv"] + alg["scores"] + alg["pv"]
            per_kernel.pop("scores"); per_kernel.pop("pv")
        log("  per-kernel (HIP events, walking the layers):")
        for k, us in per_kernel.items():
            log("    %-10s %8.2f us  %7.1f GB/s  (%.1f%% of 8 TB/s)" % (k, us, alg[k] / us / 1e3, alg[k] / us / 1e3 / 80))
        count = {k: (1 if k == "head" else cfg.n_layer) for k in per_kernel}
        if order == 1:
            names = {"qkv": "xgemv_kernel<%s, qkv> (RMSNorm in std::reduce order, Q8_0, wq|wk|wv as 8-accumulator walks, RoPE, cache write)" % tn[tt("attn_q")],
                     "scores": "xattn_scores_kernel (Dot<FP16,FP16> order, one thread per key)", "pv": "xattn_pv_kernel (softmax with std::reduce sum, P.V^T in Dot<FP16,FP16> order)",
                     "wo": "xgemv_kernel<%s, wo + residual>" % tn[tt("attn_output")], "gate_up": "xgemv_kernel<%s, gate|up + SiLU table>" % tn[tt("ffn_gate")],
                     "down": "xgemv_kernel<%s, down + residual>" % tn[tt("ffn_down")], "head": "xgemv_kernel<%s, output head>" % tn[cfg.t_out]}
        else:
            names = {"attention": "attn_layer_kernel<%s> (RMSNorm, Q8_0, wq|wk|wv, RoPE, cache write, q.K, softmax, P.V^T)" % tn[tt("attn_q")],
                     "gate_up": "wave_gemv_kernel<gate|up + SiLU>", "down": "wave_gemv_kernel<down + residual>", "wo": "wave_gemv_kernel<wo + residual>",
                     "head": "wave_gemv_kernel<output head>", "qkv": "wave_gemv_kernel<qkv>", "scores": "attn_scores_kernel", "pv": "attn_pv_kernel"}
        model_key = "%s/head_%s/order%d" % (args.model, tn[cfg.t_out], order)
        measured = traffic_db.get("kernels", {}).get(model_key, {}) if (cfg.n_embd, cfg.n_ff, cfg.n_layer) == (4096, 11008, 32) else {}

        def roof(k):
            ach = alg[k] / (per_kernel[k] * 1e-6) / 1e9
            tr = measured.get(k)
            if tr is not None and k in ("attention", "scores", "pv"):          # counted at one n_kv: scaled to this run's by the algorithmic bytes
                tr = tr["bytes"] * alg[k] / tr["algorithmic_bytes"]
            elif tr is not None:
                tr = tr["bytes"]
            return {"kernel": names.get(k, k), "bound": "hbm", "achieved": round(ach, 1), "peak": 8000.0, "unit": "GB/s", "frac": round(ach / 8000.0, 4),
                    "traffic": round(tr) if tr is not None else None, "bytes_per_launch": int(alg[k]),
                    "us_per_launch": round(per_kernel[k], 3), "launches_per_token": count[k], "share_of_step": round(per_kernel[k] * count[k] / (ev_ms * 1e3), 3)}
        dom = max(per_kernel, key=lambda k: per_kernel[k] * count[k])
        return {"order": order, "tok_s": steps / wall, "ms_per_step": wall * 1e3 / steps, "ev_ms": ev_ms, "frac": frac, "bytes_per_token": bytes_per_token, "pos": pos,
                "per_kernel": per_kernel, "roofline": roof(dom), "others": {k: roof(k) for k in per_kernel if k != dom}}

    orders = [args.order] if args.only_order else [1, 0]
    runs = {o: run_order(o) for o in orders}
    head_run = runs[orders[0]]
    pos, ev_ms = head_run["pos"], head_run["ev_ms"]
    tok_s, ms_per_step, frac, bytes_per_token = head_run["tok_s"], head_run["ms_per_step"], head_run["frac"], head_run["bytes_per_token"]
    per_kernel, roofline, roofline_others = head_run["per_kernel"], head_run["roofline"], head_run["others"]
    eng.set_order(orders[0])

    # The prompt's dominant kernels against the int8 matrix-core peak: the seven quantized GEMMs of one layer
    # (wq, wk, wv, wo: 4096 x 4096; gate, up: 11008 x 4096; down: 4096 x 11008) over the 2048 activation rows of a
    # prompt chunk, HIP events around 4 back-to-back sets.  
    gemm_roofline, gemm_roofline_o1 = None, None
    if not args.no_gemm:
        wt_g, Tg = cfg.wtype, 2048
        d_, F_ = cfg.n_embd, cfg.n_ff
        L = H.load()

        def wdev(Mg, Kg):
            wb = M.synth_tensor(wt_g, 7, "bench.gemm.%d.%d" % (Mg, Kg), Mg * Kg)
            return H.DeviceBuffer.from_numpy(wb)

        def xdev(Kg):
            xf = H.DeviceBuffer.from_numpy(np.random.default_rng(Kg).standard_normal((Tg, Kg)).astype(np.float32))
            xq_ = H.DeviceBuffer(Tg * (Kg // 32) * 34)
            H.check(L.spy_hip_quantize_q8_0(None, xf.ptr, Kg, xq_.ptr, Tg, Kg), "spy_hip_quantize_q8_0")
            H.sync()
            xf.free()
            return xq_
        w_dd, w_Fd, w_dF, x_d, x_F = wdev(d_, d_), wdev(F_, d_), wdev(d_, F_), xdev(d_), xdev(F_)
        og = H.DeviceBuffer(Tg * F_ * 4)
        layer_set = [(w_dd, x_d, d_, d_)] * 4 + [(w_Fd, x_d, F_, d_)] * 2 + [(w_dF, x_F, d_, F_)]
        e0, e1, ms = C.c_void_p(), C.c_void_p(), C.c_float()
        H.check(L.spy_hip_event_create(C.byref(e0)), "event")
        H.check(L.spy_hip_event_create(C.byref(e1)), "event")
        n_set = 4
        for timed in (False, True):
            H.check(L.spy_hip_event_record(e0, None), "record")
            for i in range(n_set):
                for (wb_, xb_, Mg, Kg) in layer_set:
                    H.check(L.spy_hip_gemm_q8_0act(None, wt_g, wb_.ptr, xb_.ptr, og.ptr, Mg, Kg, Tg, Mg), "spy_hip_gemm_q8_0act")
            H.check(L.spy_hip_event_record(e1, None), "record")
            H.sync()
        H.check(L.spy_hip_event_elapsed_ms(e0, e1, C.byref(ms)), "elapsed")
        us_set = ms.value * 1000.0 / n_set
        ops_set = 2.0 * Tg * (4 * d_ * d_ + 3 * d_ * F_)
        tops = ops_set / us_set / 1e6
        gemm_roofline = {"summation_order": 0,
                         "kernel": "gemm_q8act_kernel, the prompt GEMM of summation order 0 (NOT what the headline order's prompt runs: that is prompt_gemm_roofline): quantized GEMMs of one layer (%s weights x Q8_0 activations, int8 MFMA, per-block scales): 4 x %dx%d, 2 x %dx%d, 1 x %dx%d, %d activation rows"
                                   % ({H.Q4_0: "Q4_0", H.Q8_0: "Q8_0", H.Q4_K: "Q4_K", H.Q6_K: "Q6_K"}[wt_g], d_, d_, F_, d_, d_, F_, Tg),
                         "bound": "mfma", "achieved": round(tops, 1), "peak": INT8_PEAK / 1e12, "unit": "TOP/s", "frac": round(tops * 1e12 / INT8_PEAK, 4),
                         "ops_per_set": ops_set, "us_per_set": round(us_set, 1)}
        # what the per-block scaling leaves to the matrix cores: the kernel's inner loop on register operands only
        ceil_tops = C.c_float()
        H.check(L.spy_hip_measure_mfma_i8_scaled(None, 20000, 1, C.byref(ceil_tops)), "spy_hip_measure_mfma_i8_scaled")
        gemm_roofline["inner_loop_registers_only"] = {"achieved": round(ceil_tops.value, 1), "unit": "TOP/s", "frac_of_peak": round(ceil_tops.value * 1e12 / INT8_PEAK, 4),
                                                      "what": "one v_mfma_i32_32x32x32_i8 + the fp16 scale outer product + subtraction and fma per output, no LDS or memory"}
        log("prompt GEMMs of a layer, T = %d: %.1f us, %.0f TOP/s (%.1f%% of the int8 MFMA peak); its inner loop on register operands only: %.0f TOP/s (%.1f%%)"
            % (Tg, us_set, tops, 100 * tops * 1e12 / INT8_PEAK, ceil_tops.value, 100 * ceil_tops.value * 1e12 / INT8_PEAK))
        # The same seven products the way the prompt pass of summation order 1 runs them: spy_hip_op_matmul in the host backend's
        # order = Q8_0 quantization of the f32 activations, both operands packed as fp16, exact_gemm8p_kernel (integer sums of
        # four products from v_mfma_f32_16x16x4_4b_f16, one fma per accumulator and block on the vector units).
        gemm_roofline_o1 = None
        if cfg.wtype in (H.Q4_0, H.Q8_0):
            prev = L.spy_hip_set_exact_order(1)
            try:
                xf_d = H.DeviceBuffer.from_numpy(np.random.default_rng(d_).standard_normal((Tg, d_)).astype(np.float32))
                xf_F = H.DeviceBuffer.from_numpy(np.random.default_rng(F_).standard_normal((Tg, F_)).astype(np.float32))
                sets = [(w_dd, xf_d, d_, d_)] * 4 + [(w_Fd, xf_d, F_, d_)] * 2 + [(w_dF, xf_F, d_, F_)]
                tens = [(H.tensor(wb_, wt_g, [Kg, Mg]), H.tensor(xb_, H.F32, [Kg, Tg]), H.tensor(og, H.F32, [Mg, Tg])) for (wb_, xb_, Mg, Kg) in sets]
                need = max(L.spy_hip_op_matmul_scratch_size(C.byref(tw), C.byref(tx)) for tw, tx, _ in tens)
                scr = H.DeviceBuffer(need)
                n_set1 = 2
                for timed in (False, True):
                    H.check(L.spy_hip_event_record(e0, None), "record")
                    for i in range(n_set1):
                        for tw, tx, to in tens:
                            H.check(L.spy_hip_op_matmul(None, C.byref(tw), C.byref(tx), C.byref(to), scr.ptr, need), "spy_hip_op_matmul")
                    H.check(L.spy_hip_event_record(e1, None), "record")
                    H.sync()
                H.check(L.spy_hip_event_elapsed_ms(e0, e1, C.byref(ms)), "elapsed")
                us1 = ms.value * 1000.0 / n_set1
                tops1 = ops_set / us1 / 1e6
                gemm_roofline_o1 = {"summation_order": 1,
                                    "kernel": "exact_gemm8p_kernel + xgp_pack_kernel x 2 + Q8_0 quantization, the prompt MatMul of summation order 1 (the headline's): the same seven products "
                                              "through spy_hip_op_matmul in the host backend's order; integer sums of four products from v_mfma_f32_16x16x4_4b_f16 (fp16 matrix instructions), "
                                              "one fp32 fma per accumulator and block on the vector units",
                                    "bound": "mfma", "achieved": round(tops1, 1), "peak": INT8_PEAK / 1e12, "unit": "TOP/s", "frac": round(tops1 * 1e12 / INT8_PEAK, 4),
                                    "frac_of_fp16_mfma_peak": round(tops1 * 1e12 / 2.5e15, 4), "ops_per_set": ops_set, "us_per_set": round(us1, 1)}
                log("prompt MatMuls of a layer in summation order 1, T = %d: %.1f us, %.0f TOP/s (%.1f%% of the int8 MFMA peak, %.1f%% of the fp16 MFMA peak its matrix instructions have)"
                    % (Tg, us1, tops1, 100 * tops1 * 1e12 / INT8_PEAK, 100 * tops1 * 1e12 / 2.5e15))
                for b in (xf_d, xf_F, scr):
                    b.free()
            finally:
                L.spy_hip_set_exact_order(prev)
        for b in (w_dd, w_Fd, w_dF, x_d, x_F, og):
            b.free()

    cpu = None
    if not args.no_cpu:
        from tests import oracle_lib as O            # the checker, timed as the CPU baseline
        from tests.model_util import OracleModel
        ncpu = min(args.cpu_threads, os.cpu_count() or 1)            # the reference's configurations run with -t 8
        ora = OracleModel(cfg, tensors, nthread=ncpu)
        for il in range(cfg.n_layer):                # same cache contents as the GPU run
            ora.k_cache[il][:] = eng.read_buffer("k_cache", il, np.uint16)
            ora.v_cache[il][:] = eng.read_buffer("v_cache", il, np.uint16)
        tok = np.array([firsts[orders[0]]], np.int32)
        ora.forward(tok, fill)                        # untimed warm-up pass (cli.h:78-82)
        t0 = time.perf_counter()
        for i in range(args.cpu_steps):
            lg = ora.forward(tok, fill + i)
            tok = np.array([int(np.argmax(lg[0]))], np.int32)
        cpu_wall = time.perf_counter() - t0
        cpu = {"value": round(args.cpu_steps / cpu_wall, 3), "unit": "tok/s", "cores": ncpu, "kind": "port", "host_cpus": os.cpu_count(),
               "sample": "%d single-token passes of the same model at n_kv = %d.. (AVX2 port of Spy's host backend, OpenMP, %d threads as the reference's -t 8)"
                         % (args.cpu_steps, fill + 1, ncpu)}
        log("cpu baseline: %.3f tok/s on %d threads (%d host cpus)" % (cpu["value"], ncpu, os.cpu_count() or 0))

    head_desc = {H.Q6_K: "output head Q6_K", H.Q4_0: "output head Q4_0", H.Q8_0: "output head Q8_0", H.Q4_K: "output head Q4_K"}[cfg.t_out]
    weights_desc = {"q4_0": "Q4_0 weights, %s" % head_desc, "q8_0": "Q8_0 weights incl. head",
                    "q4_k_m": "Q4_K weights with Q6_K attn_v / ffn_down / head, 0.1 %% of the weights x 20"}[args.model] + \
                   " (seeded ~N(0, 0.02), quantized by the package's block quantizers)"
    prefill_note = {1: "prompt pass in the host backend's summation order (tiled exact kernels: integer sums from the matrix cores as floats, every accumulator of the host loops kept apart on the vector units): same logits and caches as the CPU oracle's",
                    0: "matrix-core prompt pass in the backend's own order"}
    mode_desc = {1: "host-backend summation order: logits and greedy tokens equal, bit for bit, to the CPU oracle's (Spy's host backend restated, fp contraction off; "
                    "a GCC build of Spy with its default -ffp-contract=fast fuses x * x + y in NormRMS and differs from both in the last bits)",
                 0: "this backend's own summation order (per-operator 1e-7; not token-exact)"}
    out = {
        "metric": "decode tok/s + %% HBM roofline, LLaMA-2-7B %s ctx 4096, 1xMI355X" % {"q4_0": "Q4_0", "q8_0": "Q8_0", "q4_k_m": "Q4_K_M"}[args.model],
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 dot (%s x Q8_0), fp32 accumulate, fp16 KV" % {"q4_0": "Q4_0", "q8_0": "Q8_0", "q4_k_m": "Q4_K / Q6_K"}[args.model], "data": "synthetic",
        "config": {"workload": "LLaMA-2-7B shape (32 layers, d 4096, 32 heads x 128, FFN 11008, vocab 32000), %s, " % weights_desc +
                               "f16 KV cache prefilled to %d tokens (%s), greedy single-sequence decode" % (fill, args.prefill),
                   "mode": mode_desc[orders[0]], "summation_order": orders[0],
                   "n_layer": cfg.n_layer, "n_kv_first": pos + 1, "n_kv_last": pos + steps, "bytes_per_token": int(bytes_per_token)},
        "hbm_roofline_frac": round(frac, 4), "ms_per_step_hip_events": round(ev_ms, 4),
        "prefill": {"tokens": fill, "seconds": round(prefill_s[orders[0]], 3), "tok_s": round(fill / prefill_s[orders[0]], 1), "summation_order": orders[0],
                    "note": prefill_note[orders[0]]} if args.prefill == "real" else None,
        "kernel_us": {k: round(v, 2) for k, v in per_kernel.items()},
        "roofline": roofline, "roofline_other_kernels": roofline_others, "prompt_gemm_roofline": gemm_roofline_o1 if (orders[0] == 1 and gemm_roofline_o1) else gemm_roofline,
        "prompt_gemm_roofline_other_order": gemm_roofline if (orders[0] == 1 and gemm_roofline_o1) else gemm_roofline_o1, "cpu_baseline": cpu,
    }
    if len(orders) > 1:
        o = runs[orders[1]]
        if args.prefill == "real":
            out["prefill_other_order"] = {"tokens": fill, "seconds": round(prefill_s[orders[1]], 3), "tok_s": round(fill / prefill_s[orders[1]], 1),
                                          "summation_order": orders[1], "note": prefill_note[orders[1]]}
        out["other_order"] = {"summation_order": orders[1], "mode": mode_desc[orders[1]], "value": round(o["tok_s"], 2), "unit": "tok/s",
                              "ms_per_step": round(o["ms_per_step"], 4), "hbm_roofline_frac": round(o["frac"], 4),
                              "kernel_us": {k: round(v, 2) for k, v in o["per_kernel"].items()}, "roofline": o["roofline"]}
    if load_info:
        out["gguf_load"] = load_info
    print(json.dumps(out), flush=True)
    eng.close()
    if loaded:
        loaded.close()


if __name__ == "__main__":
    main()
