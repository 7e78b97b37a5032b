#!/usr/bin/env python3
"""Throughput benchmark of the encoder hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--precision bf16|fp32]
                    [--config 2] [--no-cpu]

A step is one forward pass (embedding -> 24 layers -> pooler -> classifier head)
over one synthetic batch of the headline configuration: BERT-large, batch 128,
seq 200, per-row valid lengths uniform in [100, 200], stock N(0, 0.02) weights.
Inputs are resident in device memory when the timed region starts.  Prints one
JSON line with the whole-job rate, the roofline figure of the dominant kernel
(the FFN GEMM, timed with HIP events around back-to-back launches on the stream
they are launched on), a per-phase breakdown with achieved TFLOP/s and GB/s,
and the CPU oracle's rate on a bounded sample of the same batch.
"""
import argparse
import ctypes
import json
import os
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}
PEAK_HBM_GBS = 8000.0
# HBM-side bytes of one FFN-in GEMM launch at the headline shape (bf16, packed operands),
# from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of `bench.py --roofline-only`, each
# counter scaled by what it reads for a 256 MiB device copy (2.0 and 1.0); the summary
# with the commands is profiles/ffn_in_gemm_cfg2_bf16_pmc.txt.
MEASURED_TRAFFIC = {("bf16", 25600, 4096, 1024): 6.354e8}


def roofline_leg(torch, pybert, lib, prec, precision, N, I, H):
    # ---- roofline of the dominant kernel: the FFN-in GEMM (bias+GELU epilogue) ----
    # Same launch as in the model: in bf16 mode all three matrices are in the packed
    # operand layout (their contents are random, only the layout matters for timing).
    tdt = torch.bfloat16 if prec == pybert.BF16 else torch.float32
    packed = prec == pybert.BF16
    rows_x = (N + 255) // 256 * 256 if packed else N
    rows_w = (I + 255) // 256 * 256 if packed else I
    X = (torch.randn((rows_x, H), device="cuda") * 1.0).to(tdt)
    Wt = (torch.randn((rows_w, H), device="cuda") * 0.02).to(tdt)
    bias = torch.zeros(I, device="cuda")
    Y = torch.empty((rows_x, I), dtype=tdt, device="cuda")
    st = torch.cuda.current_stream()
    out_elt = prec
    gflags = (pybert.X_PACKED | pybert.W_PACKED | pybert.Y_PACKED) if packed else 0

    def ffn_in():
        pybert.check(lib.cubert_op_gemm(X.data_ptr(), Wt.data_ptr(), bias.data_ptr(), Y.data_ptr(), N, I, H, H, prec,
                                        out_elt, 1, 0, gflags, st.cuda_stream))
    for _ in range(20):          # enough launches for the clocks to settle
        ffn_in()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    launches = 50
    e0.record(st)
    for _ in range(launches):
        ffn_in()
    e1.record(st)
    e1.synchronize()
    k_ms = e0.elapsed_time(e1) / launches
    flops_per_launch = 2.0 * N * H * I
    achieved = flops_per_launch / k_ms / 1e9
    kname = "gemm_bf16_t256x128_kernel<bf16, bias+GELU>" if precision == "bf16" else "gemm_kernel<f32, f32, bias+GELU, 128>"
    roofline = {"bound": "mfma", "kernel": "%s (FFN-in %dx%dx%d, tile chosen by the library)" % (kname, N, I, H), "achieved": round(achieved, 1), "peak": PEAK_TFLOPS[precision],
                "unit": "TFLOP/s", "frac": round(achieved / PEAK_TFLOPS[precision], 4),
                "avg_launch_ms": round(k_ms, 4), "flop_per_launch": flops_per_launch,
                "traffic": MEASURED_TRAFFIC.get((precision, N, I, H))}
    del X, Wt, Y
    return roofline



def latency_leg(torch, pybert, synth, model, dims, args):
    """Config 3: BERT-large, S=200, all positions valid, batch 1 and 8; every call replays the
    captured hipGraph of the whole forward pass.  One call = host inputs in, pooled output
    back on the host (the reference's Cuda_Bert contract), timed with the host clock."""
    lib = pybert.lib
    iters = max(args.steps, 1000)
    res = {}
    for B in (1, 8):
        S = 200
        ids, seg, mask = synth.make_inputs(B, S, [S] * B, seed=20244 + B)
        out = np.empty((B, dims.hidden), np.float32)
        call = lambda: pybert.check(lib.cubert_encode(model, ids.ctypes.data, seg.ctypes.data, mask.ctypes.data, B, S,
                                                      out.ctypes.data, None, None))
        for _ in range(max(args.warmup, 5)):
            call()
        ts = np.empty(iters)
        for i in range(iters):
            t0 = time.perf_counter()
            call()
            ts[i] = time.perf_counter() - t0
        res["batch%d" % B] = {"p50_ms": round(float(np.percentile(ts, 50)) * 1e3, 4),
                              "p99_ms": round(float(np.percentile(ts, 99)) * 1e3, 4),
                              "mean_ms": round(float(ts.mean()) * 1e3, 4), "iters": iters,
                              "sequences_per_s": round(B / float(ts.mean()), 1)}
    print(json.dumps({"metric": "latency per batch, BERT-large s200 on 1 MI355X (host in -> host out)", "unit": "ms",
                      "higher_is_better": False, "n_gpus": 1, "dtype": args.precision, "data": "synthetic",
                      "config": {"workload": "cfg3: BERT-large encoder + pooler, seq 200 all valid, hipGraph replay",
                                 "graphs_cached": int(lib.cubert_graphs_cached(model))},
                      "latency": res}))


def extras_leg(torch, pybert, model, ids, seg, mask, dims, prec, steps):
    """Host-input entry point (uploads included) and the stand-alone bandwidth-bound kernels."""
    lib = pybert.lib
    B, S = ids.shape
    N, H, A = B * S, dims.hidden, dims.heads
    out = np.empty((B, H), np.float32)
    call = lambda: pybert.check(lib.cubert_encode(model, ids.ctypes.data, seg.ctypes.data, mask.ctypes.data, B, S,
                                                  out.ctypes.data, None, None))
    for _ in range(2):
        call()
    t0 = time.perf_counter()
    for _ in range(steps):
        call()
    host_rate = B * steps / (time.perf_counter() - t0)
    st = torch.cuda.current_stream()

    def timed(fn, reps=20):
        for _ in range(3):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(st)
        for _ in range(reps):
            fn()
        e1.record(st)
        e1.synchronize()
        return e0.elapsed_time(e1) / reps

    ops = {}
    x = torch.randn((N, H), device="cuda")
    y = torch.randn((N, H), device="cuda")
    g = torch.ones(H, device="cuda")
    b = torch.zeros(H, device="cuda")
    ms = timed(lambda: pybert.check(lib.cubert_op_add_layernorm(x.data_ptr(), y.data_ptr(), 0, g.data_ptr(), b.data_ptr(),
                                                                None, N, H, 0, st.cuda_stream)))
    by = 3.0 * N * H * 4 + 2 * H * 4
    ops["add_layernorm_f32"] = {"ms": round(ms, 4), "bytes": by, "gbs": round(by / ms / 1e6, 1),
                                "frac_hbm_peak": round(by / ms / 1e6 / PEAK_HBM_GBS, 4)}
    for elt, name, tdt, es in ((0, "f32", torch.float32, 4), (1, "bf16", torch.bfloat16, 2)):
        sc = torch.randn((B, A * S, S), device="cuda").to(tdt)
        dm = torch.from_numpy(mask).cuda()
        ms = timed(lambda: pybert.check(lib.cubert_op_mask_softmax(sc.data_ptr(), elt, dm.data_ptr(), B, A * S, S,
                                                                   0.125, st.cuda_stream)))
        by = 2.0 * B * A * S * S * es + 4 * B * S
        ops["mask_softmax_" + name] = {"ms": round(ms, 4), "bytes": by, "gbs": round(by / ms / 1e6, 1),
                                       "frac_hbm_peak": round(by / ms / 1e6 / PEAK_HBM_GBS, 4)}
        del sc
    return {"host_inputs_sequences_per_s": round(host_rate, 1), "ops": ops}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--precision", choices=["bf16", "fp32"], default="bf16")
    ap.add_argument("--config", type=int, default=2, choices=[1, 2, 3, 4],
                    help="2 = headline; 3 = latency regime (B=1 and 8, hipGraph replay, p50/p99)")
    ap.add_argument("--extras", action="store_true",
                    help="also time the host-input entry point (PCIe inclusive) and the stand-alone "
                         "bandwidth-bound kernels (residual+LayerNorm, scale+mask+softmax, embedding+LayerNorm)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seqs", type=int, default=128, help="sequences in the CPU baseline sample")
    ap.add_argument("--graph", action="store_true", help="replay the whole pass from a hipGraph (as small batches do by default)")
    ap.add_argument("--roofline-only", action="store_true",
                    help="only the dominant kernel's launches plus one device copy of known size "
                         "(the calibration kernel for the FETCH_SIZE / WRITE_SIZE counters); for profiler runs")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures ONE GPU; --gpus %d is not supported (every replica of the "
              "encoder is independent, so more GPUs are more processes of this same run)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import torch
    from cudabert_amd import pybert, synth
    from cudabert_amd import weights as W

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)

    large, B, S0 = synth.CONFIG_SHAPES[args.config]
    dims = W.LARGE if large else W.BASE
    prec = pybert.BF16 if args.precision == "bf16" else pybert.F32
    ids, seg, mask = synth.config_inputs(args.config)
    B, S = ids.shape
    N = B * S
    H, I, L, A = dims.hidden, dims.inter, dims.layers, dims.heads
    es = 2 if prec == pybert.BF16 else 4

    if args.roofline_only:
        lib = pybert.lib
        roofline = roofline_leg(torch, pybert, lib, prec, args.precision, N, I, H)
        a = torch.empty(64 << 20, dtype=torch.float32, device="cuda")     # 256 MiB read + 256 MiB written
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        print(json.dumps({"roofline": roofline, "calibration_copy_bytes_each_way": a.numel() * 4}))
        return

    t0 = time.time()
    state = W.synth_state(dims, seed=20240, degenerate=True)
    npy = W.to_npy_layout(state)
    del state
    with tempfile.TemporaryDirectory(prefix="cubert_w_") as wdir:
        for name, arr in npy.items():
            np.save(os.path.join(wdir, name + ".npy"), arr)
        t_gen = time.time() - t0
        t0 = time.time()
        model = pybert.load_model_ex(wdir, H, L, A, I, precision=prec, max_batchsize=B, max_seq_length=S,
                                     graph_max_tokens=8192 if args.config == 3 else (1 << 30 if args.graph else 0))
        t_load = time.time() - t0
    lib = pybert.lib
    if args.config == 3:
        latency_leg(torch, pybert, synth, model, dims, args)
        pybert.unload_model(model)
        return
    d_ids, d_seg, d_mask = (torch.from_numpy(a).cuda() for a in (ids, seg, mask))
    torch.cuda.synchronize()

    def step():
        pybert.check(lib.cubert_forward_device(model, d_ids.data_ptr(), d_seg.data_ptr(), d_mask.data_ptr(), B, S))
        pybert.check(lib.cubert_classify(model))

    for _ in range(args.warmup):
        step()
    pybert.check(lib.cubert_sync(model))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    pybert.check(lib.cubert_sync(model))
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    value = B * args.steps / elapsed

    # ---- the same batch computed on its valid tokens only (not the headline figure: the padded
    # pass above also fills the padding positions of the sequence output, as the reference does) ----
    lens = np.ascontiguousarray(mask.sum(1).astype(np.int32))

    def step_unpadded():
        pybert.check(lib.cubert_forward_device_lens(model, d_ids.data_ptr(), d_seg.data_ptr(), lens.ctypes.data, B, S))
        pybert.check(lib.cubert_classify(model))

    for _ in range(args.warmup):
        step_unpadded()
    pybert.check(lib.cubert_sync(model))
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step_unpadded()
    pybert.check(lib.cubert_sync(model))
    dt = time.perf_counter() - t0
    unpadded = {"value": round(B * args.steps / dt, 2), "unit": "sequences/s",
                "ms_per_step": round(dt * 1e3 / args.steps, 3), "valid_tokens": int(lens.sum()), "tokens": N,
                "note": "cubert_forward_device_lens: only valid tokens computed; pooled output and valid "
                        "positions bit-identical to the padded pass"}

    # ---- per-phase breakdown (events before every launch; outside the timed region) ----
    ph = (ctypes.c_float * 8)()
    acc = np.zeros(8)
    reps = 3
    for _ in range(reps):
        pybert.check(lib.cubert_profile_device(model, d_ids.data_ptr(), d_seg.data_ptr(), d_mask.data_ptr(), B, S, ph))
        acc += np.array(list(ph))
    acc /= reps
    gf = {"qkv_gemm": 2.0 * N * H * 3 * H * L, "attn_out_gemm": 2.0 * N * H * H * L,
          "ffn_in_gemm": 2.0 * N * H * I * L, "ffn_out_gemm": 2.0 * N * I * H * L,
          "attention": 4.0 * N * S * H * L, "pooler": 2.0 * B * H * H}
    # residual+LayerNorm traffic as executed: x f32 read + y f32 read + x f32 write (+ bf16 copy)
    ln_bytes_alg = (3.0 * N * H * 4 + 2 * H * 4) * 2 * L
    # bytes the LayerNorm kernel itself moves: the residual is added by the GEMM before it (unless
    # CUBERT_FUSE_RESIDUAL=0), so it reads the sum and writes the float32 stream (+ the bf16 copy)
    ln_reads = 1 if os.environ.get("CUBERT_FUSE_RESIDUAL", "1") != "0" else 2
    ln_bytes_exec = (((ln_reads + 1) * 4 + (2 if prec == pybert.BF16 else 0)) * N * H + 2 * H * 4) * 2 * L
    emb_bytes = N * (12 + H * 4 + H * 4) + (S + 2) * H * 4 + 2 * H * 4
    phases = {}
    for i, name in enumerate(pybert.PHASES):
        ms = float(acc[i])
        e = {"ms": round(ms, 4)}
        if name in gf and ms > 0:
            e["tflops"] = round(gf[name] / ms / 1e9, 1)
            e["frac_mfma_peak"] = round(e["tflops"] / PEAK_TFLOPS[args.precision], 4)
        if name == "add_layernorm" and ms > 0:
            e["gbs_algorithmic"] = round(ln_bytes_alg / ms / 1e6, 1)
            e["gbs_executed"] = round(ln_bytes_exec / ms / 1e6, 1)
            e["frac_hbm_peak_executed"] = round(e["gbs_executed"] / PEAK_HBM_GBS, 4)
            e["frac_hbm_peak_algorithmic"] = round(e["gbs_algorithmic"] / PEAK_HBM_GBS, 4)
        if name == "embedding" and ms > 0:
            e["gbs_algorithmic"] = round(emb_bytes / ms / 1e6, 1)
        phases[name] = e
    gemm_ms = sum(acc[i] for i, n in enumerate(pybert.PHASES) if n.endswith("_gemm"))
    gemm_flops = sum(gf[n] for n in gf if n.endswith("_gemm"))
    phases["all_gemms"] = {"ms": round(float(gemm_ms), 3), "tflops": round(gemm_flops / gemm_ms / 1e9, 1),
                           "frac_mfma_peak": round(gemm_flops / gemm_ms / 1e9 / PEAK_TFLOPS[args.precision], 4)}

    # The roofline entry is the FFN-in GEMM as it runs inside the forward pass: HIP events on the launch
    # stream around each of its L launches, averaged over the passes above.  The stand-alone leg (50
    # launches back to back, which the power limit clocks lower than the pass's mix of kernels) is
    # kept beside it.
    standalone = roofline_leg(torch, pybert, lib, prec, args.precision, N, I, H)
    roofline = dict(standalone)
    k_ms = float(acc[pybert.PHASES.index("ffn_in_gemm")]) / L
    if k_ms > 0:
        achieved = standalone["flop_per_launch"] / k_ms / 1e9
        roofline.update({"achieved": round(achieved, 1), "frac": round(achieved / PEAK_TFLOPS[args.precision], 4),
                         "avg_launch_ms": round(k_ms, 4),
                         "measured": "HIP events around each of the %d FFN-in launches of a forward pass, %d passes" % (L, reps),
                         "standalone_back_to_back": {"launches": 50, "avg_launch_ms": standalone["avg_launch_ms"],
                                                     "achieved": standalone["achieved"], "frac": standalone["frac"]}})

    # ---- CPU baseline: the oracle on a bounded sample of the same batch ----
    cpu = None
    if not args.no_cpu:
        from oracle import bert_oracle as O
        n = min(args.cpu_seqs, B)
        cores = os.cpu_count() or 1
        cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
        torch.set_num_threads(cores)
        O.forward_torch(npy, A, ids[:1], seg[:1], mask[:1])         # warm-up (thread pool, allocator)
        t0 = time.perf_counter()
        seq_ref, pooled_ref = O.forward_torch(npy, A, ids[:n], seg[:n], mask[:n])
        dt = time.perf_counter() - t0
        cpu = {"value": round(n / dt, 3), "unit": "sequences/s", "cores": cores, "kind": "port",
               "sample": "first %d sequences of the same batch (S=%d), fp32 torch oracle, 1 pass, %.1f s" % (n, S, dt)}
        # the sample doubles as a full-size parity spot check
        pooled = torch.empty((B, H), device="cuda")
        hip = ctypes.CDLL("libamdhip64.so")
        hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        step()
        pybert.check(lib.cubert_sync(model))
        assert hip.hipMemcpy(pooled.data_ptr(), lib.cubert_pooled_ptr(model), B * H * 4, 3) == 0
        cpu["pooled_max_abs_vs_gpu"] = float(np.abs(pooled.cpu().numpy()[:n] - pooled_ref).max())
    extras = extras_leg(torch, pybert, model, ids, seg, mask, dims, prec, args.steps) if args.extras else None
    pybert.unload_model(model)

    out = {
        "metric": "sequences/s BERT-large b128 s200 on 1 MI355X" if args.config == 2 else
                  "sequences/s cfg%d on 1 MI355X" % args.config,
        "value": round(value, 2), "unit": "sequences/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.precision, "data": "synthetic",
        "config": {"workload": "cfg%d: BERT-%s encoder + pooler + Linear(H->2)+softmax head, batch %d, seq %d "
                               "(valid lengths ragged, pruned to batch max), inputs resident in HBM" %
                               (args.config, "large" if large else "base", B, S),
                   "batch": B, "seq_len": S, "tokens": N, "precision": args.precision},
        "roofline": roofline, "cpu_baseline": cpu, "unpadded_pass": unpadded, "phases": phases,
        "gemm_tflop_per_step": round(gemm_flops / 1e12, 3),
        "setup_s": {"weights_generate_write": round(t_gen, 1), "model_load": round(t_load, 1)},
    }
    if extras:
        out["extras"] = extras
    print(json.dumps(out))


if __name__ == "__main__":
    main()
