#!/usr/bin/env python3
"""Throughput benchmark of the encoder hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--precision bf16|fp32]
                    [--config 2] [--no-cpu]

A step is one forward pass (embedding -> 24 layers -> pooler -> classifier head)
over one synthetic batch of the headline configuration: BERT-large, batch 128,
seq 200, per-row valid lengths uniform in [100, 200], stock N(0, 0.02) weights.
Inputs are resident in device memory when the timed region starts.  Prints one
JSON line with the whole-job rate, the roofline figure of the dominant kernel
(the FFN-in GEMM, timed with HIP events on the stream it is launched on), a
per-phase breakdown with achieved TFLOP/s and GB/s, the stand-alone bandwidth
kernels, the same pass in float32 operands, the latency regime (batch 1 and 8
from a hipGraph, p50 / p99), and the CPU oracle's rate on a bounded sample of
the same batch together with the max-abs difference of the timed pass to it.
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


def measured_traffic(precision, N, I, H):
    """HBM-side bytes of one FFN-in GEMM launch at the headline shape, as recorded in
    profiles/ffn_in_gemm_cfg2_bf16_pmc.txt: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
    `bench.py --roofline-only`, each counter scaled by what it reads for a 256 MiB device copy.
    The summary names the commit it was measured at; (None, None) for any other shape."""
    if (precision, N, I, H) != ("bf16", 25600, 4096, 1024):
        return None, None
    import re
    try:
        text = open(os.path.join(ROOT, "profiles", "ffn_in_gemm_cfg2_bf16_pmc.txt")).read()
    except OSError:
        return None, None
    m = re.search(r"-> traffic ([0-9.e+]+) bytes", text)
    c = re.search(r"measured at commit ([0-9a-f]+)", text)
    return (float(m.group(1)) if m else None), (c.group(1) if c else None)


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
                "traffic": measured_traffic(precision, N, I, H)[0],
                "traffic_source": ("profiles/ffn_in_gemm_cfg2_bf16_pmc.txt (rocprofv3 --pmc, commit %s)" %
                                   measured_traffic(precision, N, I, H)[1])
                                  if measured_traffic(precision, N, I, H)[0] is not None else None}
    # Yardstick, not part of the product: the vendor library's plain GEMM (torch.matmul: no bias, no
    # GELU, row-major operands) on the same shape and the same kind of data, timed the same way.
    try:
        Xr = torch.randn((N, H), device="cuda").to(tdt)
        Wr = (torch.randn((H, I), device="cuda") * 0.02).to(tdt)
        for _ in range(20):
            torch.matmul(Xr, Wr)
        e0.record(st)
        for _ in range(launches):
            torch.matmul(Xr, Wr)
        e1.record(st)
        e1.synchronize()
        v_ms = e0.elapsed_time(e1) / launches
        roofline["vendor_library_same_shape"] = {
            "what": "torch.matmul %dx%dx%d %s, no epilogue, %d launches back to back" % (N, I, H, precision, launches),
            "avg_launch_ms": round(v_ms, 4), "achieved": round(flops_per_launch / v_ms / 1e9, 1),
            "frac": round(flops_per_launch / v_ms / 1e9 / PEAK_TFLOPS[precision], 4)}
        del Xr, Wr
    except RuntimeError as err:            # a yardstick only: its failure must not take the record down
        roofline["vendor_library_same_shape"] = {"error": str(err)[:200]}
    del X, Wt, Y
    return roofline



def latency_leg(pybert, synth, model, dims, iters, warmup):
    """Config 3: BERT-large, S=200, all positions valid, batch 1 and 8; every call replays the
    captured hipGraph of the whole forward pass.  One call = host inputs in, pooled output
    back on the host (the reference's Cuda_Bert contract), timed with the host clock."""
    lib = pybert.lib
    res = {}
    for B in (1, 8):
        S = 200
        ids, seg, mask = synth.make_inputs(B, S, [S] * B, seed=20244 + B)
        out = np.empty((B, dims.hidden), np.float32)
        call = lambda: pybert.check(lib.cubert_encode(model, ids.ctypes.data, seg.ctypes.data, mask.ctypes.data, B, S,
                                                      out.ctypes.data, None, None))
        for _ in range(max(warmup, 5)):
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
    res["graphs_cached"] = int(lib.cubert_graphs_cached(model))
    res["what"] = "cfg3: BERT-large s200 all valid, bf16, hipGraph replay; host inputs in -> pooled output on the host"
    return res


def standalone_ops(torch, pybert, mask, B, S, H, A):
    """The bandwidth-bound kernels on their own (not inside a pass): residual + LayerNorm as the model
    launches it in bf16 mode (reads the GEMM result that already holds the residual, writes the float32
    stream and the packed bf16 copy), the same with the residual read (the reference's cuApplyLayerNorm
    traffic: 3 float32 passes), and in-place scale + mask + softmax over materialised scores."""
    lib = pybert.lib
    N = B * S
    st = torch.cuda.current_stream()

    def timed(fn, reps=30):
        for _ in range(5):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(st)
        for _ in range(reps):
            fn()
        e1.record(st)
        e1.synchronize()
        return e0.elapsed_time(e1) / reps

    def entry(ms, by):
        return {"ms": round(ms, 4), "bytes": by, "gbs": round(by / ms / 1e6, 1),
                "frac_hbm_peak": round(by / ms / 1e6 / PEAK_HBM_GBS, 4)}

    ops = {}
    x = torch.randn((N, H), device="cuda")
    y = torch.randn((N, H), device="cuda")
    g = torch.ones(H, device="cuda")
    b = torch.zeros(H, device="cuda")
    xb = torch.empty(((N + 255) // 256 * 256, H), dtype=torch.bfloat16, device="cuda")
    ms = timed(lambda: pybert.check(lib.cubert_op_add_layernorm(x.data_ptr(), y.data_ptr(), 0, g.data_ptr(), b.data_ptr(),
                                                                None, N, H, 0, st.cuda_stream)))
    ops["add_layernorm_f32"] = entry(ms, 3.0 * N * H * 4 + 2 * H * 4)
    ops["add_layernorm_f32"]["what"] = "x <- LN(x + y): 2 float32 reads + 1 float32 write per element"
    ms = timed(lambda: pybert.check(lib.cubert_op_add_layernorm(x.data_ptr(), y.data_ptr(), 0, g.data_ptr(), b.data_ptr(),
                                                                xb.data_ptr(), N, H, 4 | 16, st.cuda_stream)))
    ops["layernorm_as_in_bf16_pass"] = entry(ms, (4.0 + 4.0 + 2.0) * N * H + 2 * H * 4)
    ops["layernorm_as_in_bf16_pass"]["what"] = ("x <- LN(y), residual already added by the GEMM: float32 read + float32 "
                                                "write + packed bf16 copy per element")
    dm = torch.from_numpy(mask).cuda()
    for elt, name, tdt, es in ((0, "f32", torch.float32, 4), (1, "bf16", torch.bfloat16, 2)):
        sc = torch.randn((B, A * S, S), device="cuda").to(tdt)
        ms = timed(lambda: pybert.check(lib.cubert_op_mask_softmax(sc.data_ptr(), elt, dm.data_ptr(), B, A * S, S,
                                                                   0.125, st.cuda_stream)))
        ops["mask_softmax_" + name] = entry(ms, 2.0 * B * A * S * S * es + 4 * B * S)
        del sc
    return ops


class PowerSampler:
    """Reads the socket power (hwmon power1_input, microwatts) and the shader clock (the starred
    level of pp_dpm_sclk) of card 0 every few milliseconds in a thread while a workload runs.
    Read-only sysfs files; entries are None when the box does not expose them."""

    HWMON = "/sys/class/drm/card0/device/hwmon"
    SCLK = "/sys/class/drm/card0/device/pp_dpm_sclk"

    def __init__(self):
        self.power_file = None
        try:
            for h in sorted(os.listdir(self.HWMON)):
                f = os.path.join(self.HWMON, h, "power1_input")
                if os.path.exists(f):
                    self.power_file = f
                    self.cap_file = os.path.join(self.HWMON, h, "power1_cap")
        except OSError:
            pass

    def _read(self):
        try:
            p = int(open(self.power_file).read()) / 1e6
            star = [l for l in open(self.SCLK).read().splitlines() if "*" in l]
            mhz = float(star[0].split(":")[1].strip().lower().split("mhz")[0]) if star else None
            return p, mhz
        except (OSError, ValueError, IndexError):
            return None, None

    def measure(self, fn, seconds):
        """Calls fn() repeatedly for `seconds`; returns average power / clock over the run's later 80 %."""
        import threading
        if not self.power_file:
            return None
        samples, stop = [], threading.Event()

        def loop():
            while not stop.is_set():
                samples.append((time.perf_counter(),) + self._read())
                time.sleep(0.004)
        th = threading.Thread(target=loop, daemon=True)
        th.start()
        t0 = time.perf_counter()
        n = 0
        while time.perf_counter() - t0 < seconds:
            fn()
            n += 1
        t1 = time.perf_counter()
        stop.set()
        th.join()
        sel = [(p, c) for t, p, c in samples if t0 + 0.2 * (t1 - t0) <= t <= t1 and p is not None]
        if not sel:
            return None
        try:
            cap = int(open(self.cap_file).read()) / 1e6
        except (OSError, ValueError):
            cap = None
        clocks = [c for _, c in sel if c is not None]
        return {"power_w": round(sum(p for p, _ in sel) / len(sel), 1), "power_cap_w": cap,
                "sclk_mhz": round(sum(clocks) / len(clocks), 1) if clocks else None,
                "ms_per_call": round((t1 - t0) * 1e3 / n, 4), "samples": len(sel)}


def power_leg(torch, pybert, lib, step, sync, prec, N, I, H):
    """Where the pass stands against the board's power limit: socket power and shader clock during
    the forward pass, and during the FFN-in GEMM on its own with the pass's kind of data (random)
    and with all-zero operands (no data toggling: the same schedule at the full clock)."""
    ps = PowerSampler()
    if not ps.power_file:
        return None
    out = {}

    def passes():
        for _ in range(5):
            step()
        sync()
    out["forward_pass"] = ps.measure(passes, 2.0)
    if out["forward_pass"]:
        out["forward_pass"]["ms_per_pass"] = round(out["forward_pass"].pop("ms_per_call") / 5, 3)
    if prec != pybert.BF16:
        return out
    st = torch.cuda.current_stream()
    rows = (N + 255) // 256 * 256
    bias = torch.zeros(I, device="cuda")
    Y = torch.empty((rows, I), dtype=torch.bfloat16, device="cuda")
    # Energy per launch of the FFN-in GEMM (socket power x time): the shipped launch on the pass's kind of data and on
    # zeros, and variants that move fewer bytes for the same flops -- the 256 x 256 tile (two thirds of the LDS
    # fragment traffic of the 256 x 128 tile, fewer operand fetches) and other orders of the tiles over the XCDs.
    variants = (("ffn_in_gemm_random_operands", False, 0, 0), ("ffn_in_gemm_zero_operands", True, 0, 0),
                ("ffn_in_gemm_tile256x256", False, 256, 0), ("ffn_in_gemm_xcd_contiguous_runs", False, 0, 1 << 16),
                ("ffn_in_gemm_xcd_4x2", False, 0, 3 << 16), ("ffn_in_gemm_xcd_2x4", False, 0, 5 << 16))
    for name, zero, tile, pflag in variants:
        X = (torch.zeros if zero else torch.randn)((rows, H), device="cuda").to(torch.bfloat16)
        Wt = ((torch.zeros if zero else torch.randn)((I, H), device="cuda") * 0.02).to(torch.bfloat16)

        def launches():
            for _ in range(40):
                pybert.check(lib.cubert_op_gemm(X.data_ptr(), Wt.data_ptr(), bias.data_ptr(), Y.data_ptr(), N, I, H, H,
                                                1, 1, 1, tile, 7 | pflag, st.cuda_stream))
            torch.cuda.synchronize()
        r = ps.measure(launches, 1.2)
        if r:
            ms = r.pop("ms_per_call") / 40
            r["avg_launch_ms"] = round(ms, 4)
            r["tflops"] = round(2.0 * N * H * I / ms / 1e9, 1)
            r["frac_mfma_peak"] = round(r["tflops"] / PEAK_TFLOPS["bf16"], 4)
            r["joules_per_launch"] = round(r["power_w"] * ms / 1e3, 4)
        out[name] = r
    return out


def host_input_rate(pybert, model, ids, seg, mask, H, steps):
    """Host-input entry point: uploads and the pooled-output download are inside the timed region."""
    lib = pybert.lib
    B, S = ids.shape
    out = np.empty((B, H), np.float32)
    call = lambda: pybert.check(lib.cubert_encode(model, ids.ctypes.data, seg.ctypes.data, mask.ctypes.data, B, S,
                                                  out.ctypes.data, None, None))
    for _ in range(2):
        call()
    t0 = time.perf_counter()
    for _ in range(steps):
        call()
    return round(B * steps / (time.perf_counter() - t0), 1)


def host_in_host_out_leg(pybert, wdir, dims, ids, seg, mask, steps):
    """The reference's own timing method (cuda_bert/cuda_bert.cu:140-171): inputs in host memory, Cuda_Bert-equivalent
    call, pooled output back on the host, everything inside the timed region.  Twice: with CUBERT_VARLEN=0 (the padded
    pass the reference computes) and with the shipped defaults (a pooled-only call computes valid tokens only)."""
    lib = pybert.lib
    B, S = ids.shape
    H = dims.hidden
    out = np.empty((B, H), np.float32)
    res = {"what": "cubert_encode(pooled_out only) = Cuda_Bert: host int32 inputs in, [B, hidden] float32 out, synchronous; "
                   "H2D and D2H copies inside the timed region (cuda_bert/cuda_bert.cu:140-171)", "steps": steps}
    for name, env in (("padded_as_the_reference", {"CUBERT_VARLEN": "0", "CUBERT_FIRST_TOKEN_LAST_LAYER": "0"}),
                      ("padded_first_token_last_layer", {"CUBERT_VARLEN": "0"}), ("shipped_defaults", {})):
        old = {k: os.environ.get(k) for k in env}
        os.environ.update(env)
        try:
            m = pybert.load_model_ex(wdir, dims.hidden, dims.layers, dims.heads, dims.inter, precision=pybert.BF16,
                                     max_batchsize=B, max_seq_length=S, graph_max_tokens=8192)
        finally:
            for k, v in old.items():
                if v is None:
                    del os.environ[k]
                else:
                    os.environ[k] = v
        call = lambda: pybert.check(lib.cubert_encode(m, ids.ctypes.data, seg.ctypes.data, mask.ctypes.data, B, S,
                                                      out.ctypes.data, None, None))
        for _ in range(3):
            call()
        t0 = time.perf_counter()
        for _ in range(steps):
            call()
        dt = time.perf_counter() - t0
        pybert.unload_model(m)
        res[name] = {"value": round(B * steps / dt, 2), "unit": "sequences/s", "ms_per_call": round(dt * 1e3 / steps, 3)}
    return res


def config_leg(torch, pybert, synth, wdir, dims, cfg, precision, steps):
    """Throughput of another configuration in the same record: padded pass and valid-tokens-only pass,
    inputs resident in HBM, forward + classifier head per step (as the headline figure)."""
    lib = pybert.lib
    ids, seg, mask = synth.config_inputs(cfg)
    B, S = ids.shape
    prec = pybert.BF16 if precision == "bf16" else pybert.F32
    m = pybert.load_model_ex(wdir, dims.hidden, dims.layers, dims.heads, dims.inter, precision=prec,
                             max_batchsize=B, max_seq_length=S, graph_max_tokens=0)
    d_ids, d_seg, d_mask = (torch.from_numpy(a).cuda() for a in (ids, seg, mask))
    lens = np.ascontiguousarray(mask.sum(1).astype(np.int32))
    torch.cuda.synchronize()

    def padded():
        pybert.check(lib.cubert_forward_device(m, d_ids.data_ptr(), d_seg.data_ptr(), d_mask.data_ptr(), B, S))
        pybert.check(lib.cubert_classify(m))

    def unpadded():
        pybert.check(lib.cubert_forward_device_lens(m, d_ids.data_ptr(), d_seg.data_ptr(), lens.ctypes.data, B, S))
        pybert.check(lib.cubert_classify(m))

    out = {"workload": "cfg%d: BERT-%s b%d s%d, %s, inputs resident in HBM" %
                       (cfg, "large" if dims.layers == 24 else "base", B, S, precision),
           "tokens": int(B * S), "valid_tokens": int(lens.sum()), "steps": steps}
    for name, fn in (("padded", padded), ("valid_tokens_only", unpadded)):
        for _ in range(3):
            fn()
        pybert.check(lib.cubert_sync(m))
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        pybert.check(lib.cubert_sync(m))
        dt = time.perf_counter() - t0
        out[name] = {"value": round(B * steps / dt, 1), "unit": "sequences/s", "ms_per_step": round(dt * 1e3 / steps, 3)}
    L, H, I = dims.layers, dims.hidden, dims.inter
    gemm_flops = 2.0 * B * S * L * (3 * H * H + H * H + 2 * H * I)
    out["padded"]["all_gemms_tflops_lower_bound"] = round(gemm_flops / out["padded"]["ms_per_step"] / 1e9, 1)
    pybert.unload_model(m)
    return out


def reference_test_matrix(large_dir, base_dir, n_iter=50):
    """The reference's benchmark: test(batchsize, seq_length, nIter, large, gpu) on the six shapes of
    cuda_bert/test/test.cpp:19-35, which loads the default weight directory, repeats the 11-token seed sentence,
    and prints the 99th-percentile latency and the throughput of Cuda_Bert calls (cuda_bert/cuda_bert.cu:91-180).
    Run in a child process whose working directory holds model_npy/{base,large}_uncased, in both precisions."""
    import subprocess
    shapes = [(16, 128, False), (16, 512, False), (1, 128, True), (1, 512, True), (16, 128, True), (16, 512, True)]
    res = {"what": "libcudaBERT test() = cuda_bert/cuda_bert.cu:91-180 on the shapes of cuda_bert/test/test.cpp:19-35, "
                   "nIter %d after 10 warm-up calls; host inputs in, pooled output out per call" % n_iter}
    with tempfile.TemporaryDirectory(prefix="cubert_ref_") as cwd:
        os.makedirs(os.path.join(cwd, "model_npy"))
        os.symlink(large_dir, os.path.join(cwd, "model_npy", "large_uncased"))
        os.symlink(base_dir, os.path.join(cwd, "model_npy", "base_uncased"))
        code = ("import sys; sys.path.insert(0, %r)\nfrom cudabert_amd import pybert\n" % ROOT +
                "".join("pybert.lib.test(%d, %d, %d, %s, 0)\n" % (b, s, n_iter, lg) for b, s, lg in shapes))
        for precision in ("bf16", "fp32"):
            env = dict(os.environ, CUBERT_PRECISION=precision)
            r = subprocess.run([sys.executable, "-c", code], cwd=cwd, env=env, capture_output=True, text=True, timeout=300)
            if r.returncode != 0:
                res[precision] = {"error": (r.stderr or r.stdout)[-300:]}
                continue
            import re
            p99 = re.findall(r"99 Latency : ([0-9.]+)ms", r.stdout)
            thr = re.findall(r"Throughput: ([0-9.]+) lines per second", r.stdout)
            res[precision] = [{"model": "large" if lg else "base", "batch": b, "seq": s, "p99_ms": float(p), "calls_per_s": float(t),
                               "sequences_per_s": round(float(t) * b, 1)}
                              for (b, s, lg), p, t in zip(shapes, p99, thr)]
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--precision", choices=["bf16", "fp32"], default="bf16")
    ap.add_argument("--config", type=int, default=2, choices=[1, 2, 3, 4],
                    help="2 = headline; 3 = latency regime (B=1 and 8, hipGraph replay, p50/p99)")
    ap.add_argument("--extras", action="store_true", help="also time the host-input entry point (PCIe inclusive)")
    ap.add_argument("--no-side-legs", action="store_true",
                    help="skip what the default run records beside the headline figure: the pass in the other "
                         "precision and the latency regime (config 2 only), power and clock sampling")
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
        # For profiler runs (rocprofv3 --pmc / --kernel-trace): the dominant GEMM, the two bandwidth-bound
        # kernels of the pass at this configuration's shapes, and one device copy of known size.
        lib = pybert.lib
        roofline = roofline_leg(torch, pybert, lib, prec, args.precision, N, I, H)
        st = torch.cuda.current_stream()
        tdt = torch.bfloat16 if prec == pybert.BF16 else torch.float32
        rows = (N + 255) // 256 * 256
        # residual + LayerNorm as the pass launches it: reads the GEMM result, writes the float32 stream
        # (+ the packed bf16 copy in bf16 mode)
        x = torch.randn((N, H), device="cuda")
        y = torch.randn((N, H), device="cuda")
        g, b = torch.ones(H, device="cuda"), torch.zeros(H, device="cuda")
        xb = torch.empty((rows, H), dtype=torch.bfloat16, device="cuda")
        for _ in range(20):
            pybert.check(lib.cubert_op_add_layernorm(x.data_ptr(), y.data_ptr(), 0, g.data_ptr(), b.data_ptr(),
                                                     xb.data_ptr() if prec == pybert.BF16 else None, N, H,
                                                     (4 if prec == pybert.BF16 else 0) | 16, st.cuda_stream))
        # fused attention on this configuration's ragged masks
        Sp = (S + 31) // 32 * 32
        q = torch.randn((B, A, S, 64), device="cuda").to(tdt)
        k = torch.randn((B, A, S, 64), device="cuda").to(tdt)
        vrow = prec == pybert.BF16 and S <= 512       # as in the model: V head-major like k, transposed by the kernel's LDS reads
        vt = torch.randn((B, A, S, 64) if vrow else (B, A, 64, Sp), device="cuda").to(tdt)
        madd = np.full((B, Sp), -np.inf, np.float32)
        madd[:, :S] = (1.0 - mask.astype(np.float32)) * -10000.0
        madd = torch.from_numpy(madd).cuda()
        ctx = torch.empty((rows, H), dtype=tdt, device="cuda")
        for _ in range(20):
            pybert.check(lib.cubert_op_attention(q.data_ptr(), k.data_ptr(), vt.data_ptr(), madd.data_ptr(), ctx.data_ptr(),
                                                 B, A, S, 0.125, prec, (4 if prec == pybert.BF16 else 0) | (32 if vrow else 0),
                                                 st.cuda_stream))
        a = torch.empty(64 << 20, dtype=torch.float32, device="cuda")     # 256 MiB read + 256 MiB written
        c = torch.empty_like(a)
        for _ in range(3):
            c.copy_(a)
        torch.cuda.synchronize()
        print(json.dumps({"roofline": roofline, "calibration_copy_bytes_each_way": a.numel() * 4,
                          "layernorm_launches": 20, "attention_launches": 20}))
        return

    t0 = time.time()
    state = W.synth_state(dims, seed=20240, degenerate=True)
    npy = W.to_npy_layout(state)
    del state
    wtmp = tempfile.TemporaryDirectory(prefix="cubert_w_")
    wdir = wtmp.name
    for name, arr in npy.items():
        np.save(os.path.join(wdir, name + ".npy"), arr)
    t_gen = time.time() - t0
    t0 = time.time()
    model = pybert.load_model_ex(wdir, H, L, A, I, precision=prec, max_batchsize=B, max_seq_length=S,
                                 graph_max_tokens=8192 if args.config == 3 else (1 << 30 if args.graph else 0))
    t_load = time.time() - t0
    lib = pybert.lib
    if args.config == 3:
        lat = latency_leg(pybert, synth, model, dims, max(args.steps, 1000), args.warmup)
        pybert.unload_model(model)
        wtmp.cleanup()
        print(json.dumps({"metric": "latency per batch, BERT-large s200 on 1 MI355X (host in -> host out)", "unit": "ms",
                          "higher_is_better": False, "n_gpus": 1, "dtype": args.precision, "data": "synthetic",
                          "config": {"workload": lat["what"]}, "latency": lat}))
        return
    d_ids, d_seg, d_mask = (torch.from_numpy(a).cuda() for a in (ids, seg, mask))
    torch.cuda.synchronize()
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]

    def timed_pass(mdl, steps, warmup):
        def step():
            pybert.check(lib.cubert_forward_device(mdl, d_ids.data_ptr(), d_seg.data_ptr(), d_mask.data_ptr(), B, S))
            pybert.check(lib.cubert_classify(mdl))
        for _ in range(warmup):
            step()
        pybert.check(lib.cubert_sync(mdl))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        pybert.check(lib.cubert_sync(mdl))
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    def results_of(mdl):
        """Sequence and pooled output of the last pass, copied to the host."""
        pybert.check(lib.cubert_sync(mdl))
        pooled = np.empty((B, H), np.float32)
        seq = np.empty((B, S, H), np.float32)
        assert hip.hipMemcpy(pooled.ctypes.data, lib.cubert_pooled_ptr(mdl), pooled.nbytes, 2) == 0
        assert hip.hipMemcpy(seq.ctypes.data, lib.cubert_seq_ptr(mdl), seq.nbytes, 2) == 0
        return seq, pooled

    def phase_profile(mdl, precision_name, reps=3):
        """Per-phase breakdown: one event before every launch of an eager single-stream pass."""
        e = 2 if precision_name == "bf16" else 4
        ph = (ctypes.c_float * 8)()
        acc = np.zeros(8)
        for _ in range(reps):
            pybert.check(lib.cubert_profile_device(mdl, d_ids.data_ptr(), d_seg.data_ptr(), d_mask.data_ptr(), B, S, ph))
            acc += np.array(list(ph))
        acc /= reps
        gf = {"qkv_gemm": 2.0 * N * H * 3 * H * L, "attn_out_gemm": 2.0 * N * H * H * L,
              "ffn_in_gemm": 2.0 * N * H * I * L, "ffn_out_gemm": 2.0 * N * I * H * L,
              "attention": 4.0 * N * S * H * L, "pooler": 2.0 * B * H * H}
        Sp = (S + 31) // 32 * 32
        # residual+LayerNorm, algorithmic: x read + y read + x write, float32 (the reference's kernel)
        ln_bytes_alg = (3.0 * N * H * 4 + 2 * H * 4) * 2 * L
        # bytes the LayerNorm kernel itself moves: the residual is added by the GEMM before it (unless
        # CUBERT_FUSE_RESIDUAL=0), so it reads the sum and writes the float32 stream (+ the bf16 copy)
        ln_reads = 1 if os.environ.get("CUBERT_FUSE_RESIDUAL", "1") != "0" else 2
        ln_bytes_exec = (((ln_reads + 1) * 4 + (2 if e == 2 else 0)) * N * H + 2 * H * 4) * 2 * L
        emb_bytes = N * (12 + H * 4 + H * 4) + (S + 2) * H * 4 + 2 * H * 4
        # bf16 mode, large batches: the LayerNorm runs in the epilogue of the GEMM before it
        ln_in_gemm = (e == 2 and os.environ.get("CUBERT_FUSE_LAYERNORM", "1") != "0" and
                      os.environ.get("CUBERT_FUSE_RESIDUAL", "1") != "0" and H % 256 == 0 and N >= 6144)
        # fused attention reads q, k, v and the mask rows and writes the context: its HBM bytes (a transposed V,
        # fp32 mode or S > 512, is padded to Sp key columns)
        v_pad = 0 if (e == 2 and S <= 512 and os.environ.get("CUBERT_V_ROWMAJOR", "1") != "0") else B * A * 64 * (Sp - S) * e
        att_bytes = ((3.0 * N * H + 1.0 * N * H) * e + v_pad + 4.0 * B * Sp) * L
        phases = {}
        for i, name in enumerate(pybert.PHASES):
            ms = float(acc[i])
            d = {"ms": round(ms, 4)}
            if name in gf and ms > 0:
                d["tflops"] = round(gf[name] / ms / 1e9, 1)
                d["frac_mfma_peak"] = round(d["tflops"] / PEAK_TFLOPS[precision_name], 4)
            if name == "add_layernorm" and ms > 0:
                if ln_in_gemm:
                    d["note"] = ("no LayerNorm launches in this pass: the attn-out and FFN-out GEMMs normalise in their "
                                 "epilogue (their ms include it); what is left here is the event pairs' own time")
                else:
                    d["gbs_algorithmic"] = round(ln_bytes_alg / ms / 1e6, 1)
                    d["gbs_executed"] = round(ln_bytes_exec / ms / 1e6, 1)
                    d["frac_hbm_peak_executed"] = round(d["gbs_executed"] / PEAK_HBM_GBS, 4)
                    d["frac_hbm_peak_algorithmic"] = round(d["gbs_algorithmic"] / PEAK_HBM_GBS, 4)
            if name in ("attn_out_gemm", "ffn_out_gemm") and ln_in_gemm:
                d["includes_layernorm"] = True
            if name == "attention" and ms > 0:
                # S = 200: 97 FLOP per byte, below the machine balance (312), so HBM is the roof
                d["bound"] = "hbm"
                d["gbs"] = round(att_bytes / ms / 1e6, 1)
                d["frac_hbm_peak"] = round(d["gbs"] / PEAK_HBM_GBS, 4)
            if name == "embedding" and ms > 0:
                d["gbs_algorithmic"] = round(emb_bytes / ms / 1e6, 1)
            phases[name] = d
        gemm_ms = sum(acc[i] for i, n in enumerate(pybert.PHASES) if n.endswith("_gemm"))
        gemm_flops = sum(gf[n] for n in gf if n.endswith("_gemm"))
        phases["all_gemms"] = {"ms": round(float(gemm_ms), 3), "tflops": round(gemm_flops / gemm_ms / 1e9, 1),
                               "frac_mfma_peak": round(gemm_flops / gemm_ms / 1e9 / PEAK_TFLOPS[precision_name], 4)}
        return phases, float(acc[pybert.PHASES.index("ffn_in_gemm")]) / L, gemm_flops

    elapsed = timed_pass(model, args.steps, args.warmup)
    ms_per_step = elapsed * 1e3 / args.steps
    value = B * args.steps / elapsed
    seq_gpu, pooled_gpu = results_of(model)

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

    phases, k_ms, gemm_flops = phase_profile(model, args.precision)

    # The roofline entry is the FFN-in GEMM as it runs inside the forward pass: HIP events on the launch
    # stream around each of its L launches, averaged over the passes above.  The stand-alone leg (50
    # launches back to back, which the power limit clocks lower than the pass's mix of kernels) is
    # kept beside it.
    standalone = roofline_leg(torch, pybert, lib, prec, args.precision, N, I, H)
    roofline = dict(standalone)
    if k_ms > 0:
        achieved = standalone["flop_per_launch"] / k_ms / 1e9
        roofline.update({"achieved": round(achieved, 1), "frac": round(achieved / PEAK_TFLOPS[args.precision], 4),
                         "avg_launch_ms": round(k_ms, 4),
                         "measured": "HIP events around each of the %d FFN-in launches of a forward pass, 3 passes" % L,
                         "standalone_back_to_back": {"launches": 50, "avg_launch_ms": standalone["avg_launch_ms"],
                                                     "achieved": standalone["achieved"], "frac": standalone["frac"]}})
    # The kernel with the largest share of the pass's GPU time is not that one: it is the GEMM that also adds the
    # residual and normalises (attn-out and FFN-out share it); its FFN-out launches are timed the same way.
    roofline["kernel"] = "FFN-in GEMM: " + roofline["kernel"] + "; the best of the four linears, not the time-dominant kernel (see roofline_time_dominant)"
    fo_ms = phases["ffn_out_gemm"]["ms"] / L
    ao_ms = phases["attn_out_gemm"]["ms"] / L
    fo_flops = 2.0 * N * I * H
    with_ln = bool(phases["ffn_out_gemm"].get("includes_layernorm"))
    roofline_dominant = {
        "bound": "mfma",
        "kernel": ("gemm_bf16_t256_kernel<f32, bias + residual + LayerNorm> at the FFN-out shape %dx%dx%d" % (N, H, I)) if with_ln
                  else "FFN-out GEMM %dx%dx%d (float32 result + residual)" % (N, H, I),
        "achieved": round(fo_flops / fo_ms / 1e9, 1), "peak": PEAK_TFLOPS[args.precision], "unit": "TFLOP/s",
        "frac": round(fo_flops / fo_ms / 1e9 / PEAK_TFLOPS[args.precision], 4), "avg_launch_ms": round(fo_ms, 4),
        "flop_per_launch": fo_flops, "traffic": None,
        "measured": "HIP events around each of the %d FFN-out launches of a forward pass, 3 passes" % L,
        "includes_layernorm": with_ln,
        "same_kernel_at_the_attn_out_shape": {"shape": "%dx%dx%d" % (N, H, H), "avg_launch_ms": round(ao_ms, 4),
                                              "achieved": round(2.0 * N * H * H / ao_ms / 1e9, 1),
                                              "frac": round(2.0 * N * H * H / ao_ms / 1e9 / PEAK_TFLOPS[args.precision], 4)}}
    # (vendor_library_same_shape compares with standalone_back_to_back: both are 50 launches on their own)
    ops = standalone_ops(torch, pybert, mask, B, S, H, A)
    # With the LayerNorm inside two of the GEMMs their phase times are not GEMM-only any more; the same
    # profile of a model that launches the LayerNorm kernel keeps the pure GEMM figures comparable.
    phases_unfused = None
    if phases["attn_out_gemm"].get("includes_layernorm") and not args.no_side_legs:
        os.environ["CUBERT_FUSE_LAYERNORM"] = "0"          # read when a model is created (and by phase_profile's labels)
        try:
            mu = pybert.load_model_ex(wdir, H, L, A, I, precision=prec, max_batchsize=B, max_seq_length=S, graph_max_tokens=0)
            phases_unfused, _, _ = phase_profile(mu, args.precision)
            pybert.unload_model(mu)
        finally:
            del os.environ["CUBERT_FUSE_LAYERNORM"]

    def one_pass():
        pybert.check(lib.cubert_forward_device(model, d_ids.data_ptr(), d_seg.data_ptr(), d_mask.data_ptr(), B, S))
        pybert.check(lib.cubert_classify(model))
    power = None if args.no_side_legs else power_leg(torch, pybert, lib, one_pass, lambda: pybert.check(lib.cubert_sync(model)),
                                                     prec, N, I, H)
    host_rate = host_input_rate(pybert, model, ids, seg, mask, H, args.steps) if args.extras else None
    pybert.unload_model(model)

    # ---- beside the headline: the reference's own timing method, the other configurations, its benchmark matrix ----
    host_legs = other_cfgs = ref_matrix = None
    if args.config == 2 and args.precision == "bf16" and not args.no_side_legs:
        host_legs = host_in_host_out_leg(pybert, wdir, dims, ids, seg, mask, args.steps)
        btmp = tempfile.TemporaryDirectory(prefix="cubert_wb_")
        for name, arr in W.to_npy_layout(W.synth_state(W.BASE, seed=20240, degenerate=True)).items():
            np.save(os.path.join(btmp.name, name + ".npy"), arr)
        other_cfgs = {"cfg1_bf16": config_leg(torch, pybert, synth, btmp.name, W.BASE, 1, "bf16", 200),
                      "cfg1_fp32": config_leg(torch, pybert, synth, btmp.name, W.BASE, 1, "fp32", 40),
                      "cfg4_bf16": config_leg(torch, pybert, synth, wdir, dims, 4, "bf16", 40)}
        ref_matrix = reference_test_matrix(wdir, btmp.name)
        btmp.cleanup()

    # ---- the other precision of the same configuration, and the latency regime, in the same record ----
    other_pass = latency = None
    seq_other = pooled_other = None
    if args.config == 2 and not args.no_side_legs:
        oname = "fp32" if args.precision == "bf16" else "bf16"
        oprec = pybert.F32 if oname == "fp32" else pybert.BF16
        m2 = pybert.load_model_ex(wdir, H, L, A, I, precision=oprec, max_batchsize=B, max_seq_length=S, graph_max_tokens=0)
        osteps = 5 if oname == "fp32" else args.steps
        dt = timed_pass(m2, osteps, 2)
        seq_other, pooled_other = results_of(m2)
        oph, ok_ms, oflops = phase_profile(m2, oname, reps=1 if oname == "fp32" else 3)
        other_pass = {"dtype": oname, "value": round(B * osteps / dt, 2), "unit": "sequences/s", "steps": osteps,
                      "ms_per_step": round(dt * 1e3 / osteps, 3),
                      "roofline": {"bound": "mfma", "kernel": "FFN-in GEMM %dx%dx%d inside the forward pass" % (N, I, H),
                                   "achieved": round(2.0 * N * H * I / ok_ms / 1e9, 1), "peak": PEAK_TFLOPS[oname],
                                   "unit": "TFLOP/s", "frac": round(2.0 * N * H * I / ok_ms / 1e9 / PEAK_TFLOPS[oname], 4),
                                   "avg_launch_ms": round(ok_ms, 4)},
                      "phases": oph}
        pybert.unload_model(m2)
        m3 = pybert.load_model_ex(wdir, H, L, A, I, precision=pybert.BF16, max_batchsize=8, max_seq_length=200,
                                  graph_max_tokens=8192)
        latency = latency_leg(pybert, synth, m3, dims, 1000, 10)
        pybert.unload_model(m3)
    wtmp.cleanup()

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
        # The sample doubles as a full-size parity check of the timed pass (float32 oracle on the
        # unrounded checkpoint; in bf16 mode the error includes rounding the weights to bfloat16).
        cpu["pooled_max_abs_vs_gpu"] = float(np.abs(pooled_gpu[:n] - pooled_ref).max())
        cpu["seq_max_abs_vs_gpu"] = float(np.abs(seq_gpu[:n] - seq_ref).max())
        cpu["seq_p9999_abs_vs_gpu"] = float(np.quantile(np.abs(seq_gpu[:n] - seq_ref).ravel()[::7], 0.9999))
        cpu["seq_rms_vs_gpu"] = float(np.sqrt(np.mean((seq_gpu[:n] - seq_ref) ** 2, dtype=np.float64)))
        if other_pass is not None:
            other_pass["pooled_max_abs_vs_cpu"] = float(np.abs(pooled_other[:n] - pooled_ref).max())
            other_pass["seq_max_abs_vs_cpu"] = float(np.abs(seq_other[:n] - seq_ref).max())

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
        "roofline": roofline, "roofline_time_dominant": roofline_dominant, "cpu_baseline": cpu, "unpadded_pass": unpadded,
        "phases": phases,
        "standalone_ops": ops,
        "phases_with_separate_layernorm": phases_unfused,
        "gemm_tflop_per_step": round(gemm_flops / 1e12, 3),
        "setup_s": {"weights_generate_write": round(t_gen, 1), "model_load": round(t_load, 1)},
    }
    if other_pass is not None:
        out["%s_pass" % other_pass["dtype"]] = other_pass
    if latency is not None:
        out["latency"] = latency
    if power is not None:
        out["power"] = power
    if host_rate is not None:
        out["host_inputs_sequences_per_s"] = host_rate
    if host_legs is not None:
        out["host_in_host_out"] = host_legs
    if other_cfgs is not None:
        out["other_configurations"] = other_cfgs
    if ref_matrix is not None:
        out["reference_test_matrix"] = ref_matrix
    print(json.dumps(out))


if __name__ == "__main__":
    main()
