#!/usr/bin/env python3
"""Benchmark of the GEMM -> dense-layer -> row-primitive hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extra] [--no-cpu]

Headline (the JSON line's `value`): TFLOP/s of the bf16 4096^3 GEMM C = A.B^T with f32
accumulation and f32 output, inputs resident in HBM, whole-job throughput over K launches.
A "step" is one launch of that GEMM.  The same line carries, under "extra", the other
configurations (f32 1024^3, f16 / 8192^3, tall-skinny value-net GEMMs, the fused Leduc MLP
forward in rows/s, the row primitives in GB/s), each with its own roofline fraction, and under
"cpu_baseline" the NumPy restatement timed on this box's host cores in the same run.
Every timed case is checked against the oracle after its timed loop, and the compute units' clock during the loop is
reported next to it (`shader_clock_mhz`; the matrix-pipe peak is quoted at 2400 MHz, power-limited kernels run below).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "spiral-s-ml-library_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "f32": 157.3}   # MI355X dense MFMA peaks
PEAK_HBM_GBS = 8000.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--prewarm-ms", type=float, default=300.0,
                    help="untimed device warm-up before the W warm-up steps (the clocks of an idle GPU need tens of "
                         "milliseconds of load to ramp up)")
    ap.add_argument("--no-extra", action="store_true", help="only the headline GEMM")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--only", default=None, help="run a single extra case by name (profiling aid)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one plain copy of 1 GiB (sp_map_f32 copy: 1 GiB read, 1 GiB written) so that a "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE run of this command holds a kernel of known traffic")
    ap.add_argument("--calibrate-hbm", action="store_true",
                    help="instead of the benchmark: time the library's plain copy (sp_map_f32 copy) and its full-tensor "
                         "sum (sp_reduce_sum, a pure read) on f32 tensors of 64 MiB, 256 MiB and 1 GiB and print one "
                         "JSON line; what this box sustains, to read the HBM-bound roofline fractions against")
    return ap.parse_args()


PREWARM_MS = 300.0


CLOCK = {}   # filled by time_launches: the shader clock of the last timed loop


def time_launches(fn, steps, warmup):
    """Untimed device warm-up, W untimed + K timed launches.  Returns (wall ms per step between two
    full device syncs, HIP-event ms per launch on the launch stream).  Around the K timed launches the compute
    units' cycle counter and the constant 100 MHz counter are sampled on the same stream (sp_clock_sample): their
    ratio is the clock the units ran at during the loop, left in CLOCK["mhz"]."""
    import torch
    from ml._lib import check, lib, stream_ptr
    samples = torch.zeros(2 * CLOCK_SLOTS * 2, dtype=torch.int64, device="cuda")
    t_end = time.perf_counter() + PREWARM_MS * 1e-3
    while time.perf_counter() < t_end:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    check(lib.sp_clock_sample(samples.data_ptr(), stream_ptr()))
    t0 = time.perf_counter()
    start.record()           # torch's current stream == the stream the library launches on
    for _ in range(steps):
        fn()
    stop.record()
    check(lib.sp_clock_sample(samples.data_ptr() + CLOCK_SLOTS * 16, stream_ptr()))
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    CLOCK["mhz"] = clock_mhz(samples.cpu().numpy().reshape(2, CLOCK_SLOTS, 2))
    return wall, start.elapsed_time(stop) / steps


CLOCK_SLOTS = 32768      # slots of one sp_clock_sample result: (cycles, 100 MHz ticks) per SIMD of the chip


def clock_mhz(samples):
    """Median over the SIMDs sampled both times of (cycles1 - cycles0) / (ticks1 - ticks0) * 100 MHz from two
    sp_clock_sample results (every compute unit's cycle counter runs from a start of its own: slot by slot)."""
    import numpy as np
    first, last = samples[0].astype(np.int64), samples[1].astype(np.int64)
    both = (first[:, 1] != 0) & (last[:, 1] > first[:, 1])
    if not both.any():
        return None
    mhz = (last[both, 0] - first[both, 0]) / (last[both, 1] - first[both, 1]) * 100.0
    return round(float(np.median(mhz)), 1)


NOMINAL_MHZ = 2400.0     # the clock the published peak rates are quoted at


def roofline_mfma(flops, ms, dtype):
    achieved = flops / (ms * 1e-3) / 1e12
    return {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_TFLOPS[dtype], "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_TFLOPS[dtype], 4), "traffic": None}


def roofline_hbm(nbytes, ms):
    achieved = nbytes / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": round(achieved / PEAK_HBM_GBS, 4), "traffic": None}


def best_of(fn, reps):
    fn()
    best = float("inf")
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        best = min(best, time.perf_counter() - t0)
    return best


def calibrate_hbm(steps, warmup):
    """Copy and read rates of the library's own streaming kernels (HIP-event time per launch)."""
    import torch
    from ml._lib import check, lib, ptr, stream_ptr
    torch.cuda.set_device(0)
    out = {}
    ws = torch.zeros(lib.sp_reduce_workspace_bytes(), dtype=torch.uint8, device="cuda")
    res = torch.empty(4, dtype=torch.float32, device="cuda")
    for mib in (64, 256, 1024):
        n = mib * (1 << 20) // 4
        x = torch.rand(n, dtype=torch.float32, device="cuda")
        y = torch.empty_like(x)
        _, ev = time_launches(lambda: check(lib.sp_map_f32(0, ptr(x), ptr(y), n, stream_ptr())), steps, warmup)
        out["copy_%dMiB" % mib] = {"ms": round(ev, 5), "gbs": round(2 * 4 * n / (ev * 1e-3) / 1e9, 1)}
        _, ev = time_launches(lambda: check(lib.sp_reduce_sum(0, ptr(x), ptr(res), n, ptr(ws), ws.numel(), stream_ptr())),
                              steps, warmup)
        out["read_%dMiB" % mib] = {"ms": round(ev, 5), "gbs": round(4 * n / (ev * 1e-3) / 1e9, 1)}
        _, ev = time_launches(lambda: y.fill_(1.0), steps, warmup)      # write only (torch's fill kernel)
        out["write_%dMiB" % mib] = {"ms": round(ev, 5), "gbs": round(4 * n / (ev * 1e-3) / 1e9, 1)}
        del x, y
        torch.cuda.empty_cache()
    print(json.dumps({"hbm_calibration": out, "unit": "GB/s", "peak": PEAK_HBM_GBS, "steps": steps, "warmup": warmup,
                      "kernels": "sp_map_f32(copy): n bytes read + n written; sp_reduce_sum(f32): n bytes read; "
                                 "torch.Tensor.fill_: n bytes written"}))


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (every GPU box here has one GPU "
              "and the path has no collective step)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from ml import layers, matmul, primitives
    from oracle import gemm as ogemm, layers as olayers, row_ops as orow

    global PREWARM_MS
    PREWARM_MS = args.prewarm_ms
    if args.calibrate_hbm:
        calibrate_hbm(args.steps, args.warmup)
        return
    torch.cuda.set_device(0)
    TD = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
    dev = lambda x, t=None: torch.from_numpy(np.ascontiguousarray(x)).cuda().to(t or torch.from_numpy(x).dtype)
    K, W = args.steps, args.warmup

    def gemm_inputs(seed, m, n, k, dtype):
        rng = np.random.default_rng(seed)
        scale = np.float32(1.0 / np.sqrt(k)) if dtype != "f32" else np.float32(1.0)
        a = ogemm.round_to(rng.standard_normal((m, k), dtype=np.float32) * scale, dtype)
        b = ogemm.round_to(rng.standard_normal((n, k), dtype=np.float32) * scale, dtype)
        return a, b

    def gemm_case(seed, m, n, k, dtype, out="f32", bias_relu=False, steps=K, warmup=W):
        a, b = gemm_inputs(seed, m, n, k, dtype)
        ad, bd = dev(a, TD[dtype]), dev(b, TD[dtype])
        c = torch.empty((m, n), dtype=TD[out], device="cuda")
        bias_h = np.random.default_rng(seed + 1).standard_normal(n, dtype=np.float32) if bias_relu else None
        bias = dev(bias_h) if bias_relu else None
        fn = lambda: matmul.matmul_abt(ad, bd, c, bias=bias, relu=bias_relu)
        wall, ev = time_launches(fn, steps, warmup)
        mhz = CLOCK["mhz"]
        # what was timed is checked: a block of 64 sampled rows of the last launch's C against the oracle
        rows = np.random.default_rng(seed + 2).choice(m, size=min(m, 64), replace=False)
        rows.sort()
        want = ogemm.gemm_abt(a[rows], b)
        if bias_relu:
            want = np.maximum(want + bias_h, 0)
        got = c[torch.from_numpy(rows).cuda()].float().cpu().numpy()
        err = ogemm.rel_frobenius(got, want)
        assert err < (1e-5 if dtype == "f32" else 3e-3), "bench GEMM output drifted from the oracle: %g" % err
        flops = 2.0 * m * n * k
        es_in, es_out = (4 if dtype == "f32" else 2), (4 if out == "f32" else 2)
        nbytes = es_in * (m * k + n * k) + es_out * m * n + (4 * n if bias_relu else 0)
        t_mfma = flops / (PEAK_TFLOPS[dtype] * 1e12)
        t_mem = nbytes / (PEAK_HBM_GBS * 1e9)
        # the roofline fraction comes from the same clock as the throughput figure: wall time between two device syncs
        roof = roofline_mfma(flops, wall, dtype) if t_mfma >= t_mem else roofline_hbm(nbytes, wall)
        if roof["bound"] == "mfma":
            # the published peak assumes the nominal clock; a power-limited kernel runs below it, and this is the
            # fraction of what the matrix pipes could do at the clock they were actually given
            roof["frac_at_measured_clock"] = round(roof["frac"] * NOMINAL_MHZ / mhz, 4) if mhz else None
        res = {"ms": round(ev, 5), "wall_ms": round(wall, 5), "tflops": round(flops / (wall * 1e-3) / 1e12, 2),
               "gbs": round(nbytes / (wall * 1e-3) / 1e9, 1), "roofline": roof, "seed": seed, "shader_clock_mhz": mhz,
               "checked_rel_frobenius": float("%.3g" % err),
               "tile": matmul.matmul_config_tf32(False, True, m, n, k, TD[dtype])}
        return res, (a, b)

    if args.calibrate_copy:
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")
        primitives.map("copy", src)
        torch.cuda.synchronize()
        del src
        torch.cuda.empty_cache()

    # ---------------- headline: bf16 4096^3, f32 accumulate, f32 out ----------------
    flops = 2.0 * 4096 ** 3
    if args.only:   # profiling aid: only the named extra case runs, the headline fields stay empty
        head, a, b = {"tflops": None, "wall_ms": None, "roofline": None, "tile": None, "shader_clock_mhz": None}, None, None
    else:
        head, (a, b) = gemm_case(2, 4096, 4096, 4096, "bf16")

    cpu = None
    if not args.no_cpu and not args.only:
        t = best_of(lambda: np.matmul(a, b.T), 3)
        blas = {"vendor": None, "version": None, "threads": None}
        try:   # which BLAS np.matmul ran on and with how many threads
            from threadpoolctl import threadpool_info
            pools = [p for p in threadpool_info() if p.get("user_api") == "blas"]
            if pools:
                blas = {"vendor": pools[0].get("internal_api"), "version": pools[0].get("version"),
                        "threads": pools[0].get("num_threads")}
        except Exception:   # informational only
            pass
        cpu = {"value": round(flops / t / 1e12, 4), "unit": "TFLOP/s",
               "cores": blas["threads"] or len(os.sched_getaffinity(0)),
               "kind": "port", "sample": "full 4096^3 problem, np.matmul(A32, B32.T) in f32 on the bf16-rounded "
               "inputs, 1 warm-up + best of 3", "blas": blas, "cpus_allowed": len(os.sched_getaffinity(0)),
               "os_cpu_count": os.cpu_count()}
    del a, b

    extra = {}
    cases = []
    if not args.no_extra or args.only:
        cases = [
            ("gemm_f32_1024", lambda: gemm_case(1, 1024, 1024, 1024, "f32")[0]),
            ("gemm_bf16_4096_bf16out", lambda: gemm_case(2, 4096, 4096, 4096, "bf16", "bf16")[0]),
            ("gemm_f16_4096", lambda: gemm_case(2, 4096, 4096, 4096, "f16")[0]),
            ("gemm_bf16_8192", lambda: gemm_case(3, 8192, 8192, 8192, "bf16", steps=max(3, K // 5), warmup=2)[0]),
            ("gemm_bf16_65536x256x256", lambda: gemm_case(4, 65536, 256, 256, "bf16")[0]),
            ("gemm_bf16_65536x1024x512", lambda: gemm_case(5, 65536, 1024, 512, "bf16")[0]),
            ("gemm_bf16_65536x256x2048", lambda: gemm_case(6, 65536, 256, 2048, "bf16")[0]),
            ("gemm_bf16_65536x256x256_bias_relu", lambda: gemm_case(4, 65536, 256, 256, "bf16", bias_relu=True)[0]),
            ("gemm_bf16_65536x1024x512_bias_relu", lambda: gemm_case(5, 65536, 1024, 512, "bf16", bias_relu=True)[0]),
        ]

        def mlp_case(packed=True, batches=1):
            """batches = 1: one launch per batch of 16384 rows, back to back.  batches > 1: ONE launch over that many
            batches of 16384 rows (the other timing mode the workload's definition allows); the per-batch time is then
            free of what lies between two launches."""
            rng = np.random.default_rng(7)
            dims = [32, 256, 256, 256, 3]
            batch = 16384 * batches
            x = (rng.random((batch, 32)) < 0.2).astype(np.float32)
            ws = [ogemm.round_to(olayers.weight_init(rng, o, i), "f16") for i, o in zip(dims[:-1], dims[1:])]
            u = (1 - rng.random(batch, dtype=np.float32)).astype(np.float32)
            xd, wd, ud = dev(x, torch.float16), [dev(w, torch.float16) for w in ws], dev(u)
            policy = torch.empty((batch, 3), dtype=torch.float32, device="cuda")
            action = torch.empty((batch,), dtype=torch.int32, device="cuda")
            import ctypes as C
            from ml import _lib
            wp = (C.c_void_p * 4)(*[w.data_ptr() for w in wd])
            dp = (C.c_int32 * 5)(*dims)
            if packed:
                # the weights are packed into MFMA operand order ONCE, outside the timed region (a change of layout
                # made when the weights are set, like a transpose at model load); every timed step is one
                # sp_mlp_forward_packed launch that reads nothing but the packed buffer, x and u
                pk = layers.pack_weights(wd)
                call = (_lib.SP_F16, _lib.ptr(xd), 4, _lib.ptr(pk.buffer), pk.buffer.numel(), None, dp, _lib.ptr(ud), None,
                        _lib.ptr(policy), _lib.ptr(action), None, batch, _lib.HEAD_SOFTMAX_RM, 0)
                fn = lambda: _lib.check(_lib.lib.sp_mlp_forward_packed(*call, _lib.stream_ptr()))
            else:
                call = (_lib.SP_F16, _lib.ptr(xd), 4, wp, None, dp, _lib.ptr(ud), None, _lib.ptr(policy), _lib.ptr(action),
                        None, batch, _lib.HEAD_SOFTMAX_RM, 0)
                fn = lambda: _lib.check(_lib.lib.sp_mlp_forward(*call, _lib.stream_ptr()))
            wall, ev = time_launches(fn, max(K, 200) if batches == 1 else max(K // 4, 20), W)
            sample = slice(0, batch, max(1, batch // 16384))           # every batches-th row: 16384 rows checked
            want_p, want_a, _ = olayers.mlp_forward(x[sample], ws, u=u[sample])
            got_p = policy.cpu().numpy()[sample]
            assert ogemm.rel_frobenius(got_p, want_p) < 3e-3, "bench MLP output drifted from the oracle"
            assert (action.cpu().numpy()[sample] == orow.discrete_sampling(got_p, u[sample])).all(), "bench MLP actions"
            fl = 2.0 * 16384 * sum(i * o for i, o in zip(dims[:-1], dims[1:]))
            per = ev / batches
            res = {"ms": round(per, 5), "wall_ms": round(wall / batches, 5), "rows_per_s": round(16384 / (per * 1e-3), 1),
                   "roofline": roofline_mfma(fl, per, "f16"), "seed": 7, "shader_clock_mhz": CLOCK["mhz"],
                   "weights": "packed once before the timed region (sp_mlp_pack_weights + sp_mlp_forward_packed)" if packed
                   else "row-major, as the reference keeps them (sp_mlp_forward: the drop-in call)",
                   "timing": "mean over back-to-back launches of one 16384-row batch each, between two HIP events" if batches == 1
                   else "ONE launch over %d batches of 16384 rows (%d rows), mean over back-to-back launches between two HIP "
                        "events, divided by %d: time per 16384-row batch without what lies between two launches"
                        % (batches, batch, batches)}
            if batches > 1:
                res["launch_ms"] = round(ev, 5)
                res["batches_per_launch"] = batches
            if not args.no_cpu and batches == 1:
                t = best_of(lambda: olayers.mlp_forward(x, ws, u=u), 3)
                res["cpu_rows_per_s"] = round(batch / t, 1)
            return res

        def rows_case(materialise):
            rng = np.random.default_rng(8)
            rows, cols = 65536, 256
            x = (rng.standard_normal((rows, cols), dtype=np.float32) * np.float32(2)).astype(np.float32)
            u = (1 - rng.random(rows, dtype=np.float32)).astype(np.float32)
            xd, ud = dev(x), dev(u)
            want = ("rowmax", "rowsum", "argmax", "sample") + (("probs", "cdf") if materialise else ())
            outs = {}
            for name in want:
                shape = (rows, cols) if name in ("probs", "cdf") else (rows,)
                outs[name] = torch.empty(shape, dtype=torch.int32 if name in ("argmax", "sample") else torch.float32,
                                         device="cuda")
            from ml._lib import check, lib, ptr, stream_ptr
            fn = lambda: check(lib.sp_row_ops(ptr(xd), ptr(ud), ptr(outs["rowmax"]), ptr(outs["rowsum"]),
                                              ptr(outs.get("probs")), ptr(outs.get("cdf")), ptr(outs["argmax"]),
                                              ptr(outs["sample"]), rows, cols, 0, stream_ptr()))
            wall, ev = time_launches(fn, K, W)
            nbytes = rows * cols * 4 * (3 if materialise else 1) + rows * 4 * 5
            res = {"ms": round(ev, 5), "wall_ms": round(wall, 5), "rows_per_s": round(rows / (ev * 1e-3), 1),
                   "roofline": roofline_hbm(nbytes, ev), "seed": 8, "sigma": 2.0, "shader_clock_mhz": CLOCK["mhz"]}
            assert (outs["argmax"].cpu().numpy() == orow.argmax(x)).all(), "bench row ops: argmax"
            assert (outs["rowmax"].cpu().numpy() == x.max(axis=1)).all(), "bench row ops: row maximum"
            if materialise:
                # what was timed is checked: argmax exact, the sampled index exact given the kernel's own running sums,
                # and how many rows would sample another index under a left-to-right running sum of the same
                # probabilities (the kernel's association is a fixed tree; the two differ where u * m falls between them)
                probs, cdf = outs["probs"].cpu().numpy(), outs["cdf"].cpu().numpy()
                sample = outs["sample"].cpu().numpy()
                assert (outs["argmax"].cpu().numpy() == orow.argmax(x)).all(), "bench row ops: argmax"
                assert (sample == orow.discrete_sampling(probs, u, cdf=cdf)).all(), "bench row ops: sampled index"
                seq = orow.discrete_sampling(probs, u, order="sequential")
                res["rows_sampling_differently_under_sequential_cdf"] = int((seq != sample).sum())
                res["rows"] = rows
            if not args.no_cpu and materialise:
                def cpu_rows():
                    p = orow.softmax(x)
                    cdf = orow.inclusive_scan_sum(p)
                    return orow.argmax(x), orow.discrete_sampling(p, u, cdf=cdf)
                t = best_of(cpu_rows, 2)
                res["cpu_gbs"] = round(nbytes / t / 1e9, 2)
            return res

        def elementwise_case(kind):
            # map / reduce / grid_transpose_snd of ml/primitives.spi on the row-primitive tensor shape
            rng = np.random.default_rng(9)
            rows, cols = 65536, 256
            x = rng.standard_normal((rows, cols), dtype=np.float32)
            xd = dev(x)
            if kind == "map_relu":
                out = torch.empty_like(xd)
                fn = lambda: primitives.map("relu", xd, out=out)
                nbytes = 2 * x.nbytes
            elif kind == "reduce_sum":
                from ml._lib import check, lib, ptr, stream_ptr
                ws = torch.zeros(lib.sp_reduce_workspace_bytes(), dtype=torch.uint8, device="cuda")
                out = torch.empty(4, dtype=torch.float32, device="cuda")
                fn = lambda: check(lib.sp_reduce_sum(0, ptr(xd), ptr(out), xd.numel(), ptr(ws), ws.numel(), stream_ptr()))
                nbytes = x.nbytes + 4
            else:
                out = torch.empty((cols, rows), dtype=torch.float32, device="cuda")
                fn = lambda: primitives.transpose_snd(xd, out=out)
                nbytes = 2 * x.nbytes
            wall, ev = time_launches(fn, K, W)
            got = out.cpu().numpy()
            if kind == "map_relu":
                assert (got == np.maximum(x, np.float32(0))).all(), "bench map: output differs from the oracle"
            elif kind == "reduce_sum":
                want = float(x.sum(dtype=np.float64))
                assert abs(float(got[0]) - want) <= 1e-5 * float(np.abs(x).sum(dtype=np.float64)), "bench reduce: sum"
            else:
                assert (got == x.T).all(), "bench transpose: output differs from the oracle"
            return {"ms": round(ev, 5), "wall_ms": round(wall, 5), "roofline": roofline_hbm(nbytes, ev), "seed": 9,
                    "shader_clock_mhz": CLOCK["mhz"]}

        def graph_case():
            # The same policy step through the reference's host surface: a layer graph (input -> matmul/relu x3 ->
            # matmul -> masked softmax + sample, device Philox uniforms) run by layers.graph_run_host.  The head is 64
            # wide with 3 valid columns because the reference's row ops need 16-byte rows.
            q = layers.blocks_per_grid()
            batch = 16384
            g = layers.pipe(layers.input("input", (q, batch // q, 32), "f16"), layers.matmul((32, 256)), layers.relu,
                            layers.matmul((256, 256)), layers.relu, layers.matmul((256, 256)), layers.relu,
                            layers.matmul((256, 64)), layers.masked_softmax_and_discrete_sample(3))
            m = layers.create_model(g)
            rng = np.random.default_rng(10)
            xin = layers.key_extract(m, "input")
            xin.copy_(dev((rng.random(tuple(xin.shape)) < 0.2).astype(np.float32), torch.float16))
            for _, t, _ in layers.extract_layers_(m, layers.weight_id()):
                t.copy_(dev(olayers.weight_init(rng, t.shape[0], t.shape[1]), torch.float16))
            fn = lambda: layers.graph_run_host(m, static_weights=True)
            wall, ev = time_launches(fn, max(K, 200), W)
            probs, acts = layers.graph_extract(m)
            probs, acts = probs.cpu().numpy().reshape(batch, 64), acts.cpu().numpy().reshape(batch)
            assert (probs[:, 3:] == 0).all() and np.abs(probs.sum(axis=1) - 1).max() < 1e-5, "bench graph: policy rows"
            assert ((acts >= 0) & (acts < 3)).all() and (probs[np.arange(batch), acts] > 0).all(), "bench graph: actions"
            fl = 2.0 * batch * (32 * 256 + 256 * 256 + 256 * 256 + 256 * 64)
            return {"ms": round(ev, 5), "wall_ms": round(wall, 5), "rows_per_s": round(batch / (ev * 1e-3), 1),
                    "roofline": roofline_mfma(fl, ev, "f16"), "seed": 10,
                    "shader_clock_mhz": CLOCK["mhz"],
                    "timing": "mean over back-to-back graph_run_host(static_weights=True) calls: one fused-MLP launch each, "
                              "on weights packed once when the plan is built; every run draws its own Philox uniforms "
                              "inside the kernel (nothing is carried over from run to run but the packed weights)"}

        def ensemble_case():
            # The reference's own policy network (game/leduc/model_cem.spi:55-63) through its host surface: a layer
            # graph of E = 32 members, 128 -> 64 -> relu -> 64, masked regret matching over 3 of 64 columns, f32, on
            # blocks_per_grid x 256 rows; graph_run_host(model, {"ensemble": 32}) is ONE fused launch.
            ens, q, w = 32, layers.blocks_per_grid(), 256
            probs = layers.apply("ensemble", layers.input("output_probs", (ens, q, w, 64)))
            net = layers.pipe(layers.input("input", (q, w, 128)), layers.matmul_ensemble_with_adjoint((ens, 128, 64)),
                              layers.relu, layers.matmul_ensemble_with_adjoint((ens, 64, 64)))
            m = layers.create_model(layers.masked_regret_matching_(3, probs, net))
            rng = np.random.default_rng(11)
            xin = layers.key_extract(m, "input")
            x = rng.standard_normal(tuple(xin.shape), dtype=np.float32)
            xin.copy_(dev(x))
            ws = []
            for t in layers.key_extract_list(m, "weights"):
                ws.append(rng.standard_normal(tuple(t.shape), dtype=np.float32) * np.float32(0.1))
                t.copy_(dev(ws[-1]))
            rows = q * w
            fn = lambda: layers.graph_run_host(m, {"ensemble": ens})
            wall, ev = time_launches(fn, max(K // 2, 20), W)
            mhz = CLOCK["mhz"]
            got = layers.key_extract(m, "output_probs").cpu().numpy().reshape(ens, rows, 64)
            sample = slice(0, rows, max(1, rows // 512))
            for e in (0, ens - 1):                                # what was timed is checked: two members, 512 rows each
                want, _, _ = olayers.mlp_forward(x.reshape(rows, 128)[sample], [ws[0][e], ws[1][e]], None,
                                                 olayers.HEAD_REGRET_MATCHING, None, None, 3)
                assert ogemm.rel_frobenius(got[e][sample], want) < 1e-5, "bench ensemble output drifted from the oracle"
            slow = lambda: layers.graph_run_host(m, {"ensemble": ens}, fuse=False)
            _, ev_nodes = time_launches(slow, max(K // 10, 5), 2)
            # flops the masked graph needs: the second layer only for the 3 columns the mask keeps (the reference's
            # node-by-node pass multiplies all 64 and masks afterwards: 2 * (128 * 64 + 64 * 64) per member-row)
            fl = 2.0 * rows * ens * (128 * 64 + 64 * 3)
            roof = roofline_mfma(fl, ev, "f32")
            roof["frac_counting_all_64_columns"] = round(2.0 * rows * ens * (128 * 64 + 64 * 64) / (ev * 1e-3) / 1e12 / PEAK_TFLOPS["f32"], 4)
            return {"ms": round(ev, 5), "wall_ms": round(wall, 5), "rows_per_s": round(rows * ens / (ev * 1e-3), 1),
                    "roofline": roof, "seed": 11, "shader_clock_mhz": mhz,
                    "rows": rows, "members": ens, "node_by_node_ms": round(ev_nodes, 5),
                    "timing": "mean over back-to-back graph_run_host(model, {ensemble: 32}) calls, one sp_mlp_forward_ensemble "
                              "launch each; node_by_node_ms: the same graph with fuse=False (batched GEMM, relu map, "
                              "batched GEMM, row map: four launches); rows_per_s counts member-rows"}

        def cfr_case():
            # The reference's CFR model (game/leduc/model_cfr.spi:56-61): E = 4 members, 128 -> 128, binarize into 4096
            # worlds, f32, on blocks_per_grid x 256 rows; graph_run_host(model, {"ensemble": 4}) is ONE launch that computes
            # the 32 columns the hash can see and never writes the product.
            ens, q, w = 4, layers.blocks_per_grid(), 256
            world = layers.apply("ensemble", layers.input("output_world_id", (ens, q, w), "int"))
            net = layers.pipe(layers.input("input", (q, w, 128)), layers.matmul_ensemble((ens, 128, 128)))
            m = layers.create_model(layers.binarize_(1 << 12, world, net))
            rng = np.random.default_rng(12)
            xin = layers.key_extract(m, "input")
            x = rng.standard_normal(tuple(xin.shape), dtype=np.float32)
            xin.copy_(dev(x))
            wt = layers.key_extract_list(m, "weights")[0]
            wv = rng.standard_normal(tuple(wt.shape), dtype=np.float32)
            wt.copy_(dev(wv))
            rows = q * w
            fn = lambda: layers.graph_run_host(m, {"ensemble": ens})
            wall, ev = time_launches(fn, K, W)
            mhz = CLOCK["mhz"]
            got = layers.key_extract(m, "output_world_id").cpu().numpy().reshape(ens, rows).view(np.uint32)
            sample = slice(0, rows, max(1, rows // 2048))
            for e in (0, ens - 1):                                # what was timed is checked (signs next to zero aside)
                y = ogemm.gemm_abt(x.reshape(rows, 128)[sample], wv[e])
                sure = (np.abs(y[:, :32]) > 1e-4).all(axis=1)
                assert (got[e][sample][sure] == orow.binarize(y, 1 << 12)[sure]).all(), "bench CFR hash drifted from the oracle"
            slow = lambda: layers.graph_run_host(m, {"ensemble": ens}, fuse=False)
            _, ev_nodes = time_launches(slow, max(K // 10, 5), 2)
            fl = 2.0 * rows * ens * 128 * 32               # the 32 columns the device's 32-bit shift lets the hash see
            return {"ms": round(ev, 5), "wall_ms": round(wall, 5), "rows_per_s": round(rows * ens / (ev * 1e-3), 1),
                    "roofline": roofline_mfma(fl, ev, "f32"), "seed": 12, "shader_clock_mhz": mhz, "rows": rows,
                    "members": ens, "node_by_node_ms": round(ev_nodes, 5),
                    "timing": "mean over back-to-back graph_run_host(model, {ensemble: 4}) calls, one sp_ensemble_binarize "
                              "launch each; node_by_node_ms: the same graph with fuse=False (batched GEMM over all 128 "
                              "columns, then the row hash); rows_per_s counts member-rows"}

        cases += [("ensemble_leduc_policy_e32", ensemble_case), ("ensemble_leduc_cfr_e4", cfr_case)]
        cases += [("mlp_leduc_16384", mlp_case), ("mlp_leduc_16384_rowmajor", lambda: mlp_case(False)),
                  ("mlp_leduc_16384x64_one_launch", lambda: mlp_case(True, 64)),
                  ("mlp_leduc_16384x64_one_launch_rowmajor", lambda: mlp_case(False, 64)),
                  ("layers_graph_leduc_16384", graph_case), ("row_ops_65536x256_scalars", lambda: rows_case(False)),
                  ("row_ops_65536x256_materialised", lambda: rows_case(True)),
                  ("map_relu_65536x256", lambda: elementwise_case("map_relu")),
                  ("reduce_sum_f32_65536x256", lambda: elementwise_case("reduce_sum")),
                  ("transpose_65536x256", lambda: elementwise_case("transpose"))]
    for name, fn in cases:
        if args.only and name != args.only:
            continue
        extra[name] = fn()
        torch.cuda.empty_cache()

    # The MLP's two timing modes side by side: `ms` of a one-launch-per-batch case is the launch-to-launch interval of
    # back-to-back launches; `kernel_ms` is the time per 16384-row batch inside ONE launch over 64 batches, which no
    # launch effect can touch (that launch takes the kernels of the family that keep the weights in registers).
    for single, many in (("mlp_leduc_16384", "mlp_leduc_16384x64_one_launch"),
                         ("mlp_leduc_16384_rowmajor", "mlp_leduc_16384x64_one_launch_rowmajor")):
        if single in extra and many in extra:
            extra[single]["kernel_ms"] = extra[many]["ms"]
            extra[single]["kernel_ms_from"] = many

    info = None
    try:
        from ml._lib import device_info
        info = device_info()
    except Exception as e:  # the device query is informational only
        info = {"error": str(e)}

    # HBM-side traffic per launch, measured separately with rocprofv3 --pmc (the counters cannot be read from inside
    # this process); profiles/traffic.json holds the scaled figures together with a hash of the kernel source each
    # was measured on.  A figure is only copied into the line while that source is unchanged: after an edit it is
    # stale until the counters have been collected again, and the line says so instead.
    try:
        import hashlib
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            measured = json.load(f)

        def source_hash(src):
            """sha256 over a kernel source and the headers of its directory, in name order."""
            csrc = os.path.join(ROOT, "spiral-s-ml-library_amd", "csrc")
            h = hashlib.sha256()
            for name in [src] + sorted(n for n in os.listdir(csrc) if n.endswith(".h")):
                with open(os.path.join(csrc, name), "rb") as fh:
                    h.update(fh.read())
            return h.hexdigest()

        def source_unchanged(entry):
            src = entry.get("source")
            return bool(src) and source_hash(src) == measured.get("source_sha256", {}).get(src)

        for name, res in [("headline", head)] + list(extra.items()):
            if name in measured and res.get("roofline") is not None:
                if source_unchanged(measured[name]):
                    res["roofline"]["traffic"] = measured[name]["traffic_bytes"]
                else:
                    res["roofline"]["traffic_stale"] = "%s changed since profiles/traffic.json was measured" % measured[name].get("source")
    except (OSError, KeyError, ValueError):
        pass

    # `value`, `ms_per_step` and `roofline` come from the same clock (wall time between two device syncs around the
    # K launches): value = roofline.achieved = 2 * 4096^3 / ms_per_step.  `event_ms_per_step` is the same interval
    # between two HIP events on the launch stream; the two differ by the host's share of a launch.
    # `mlp_rows_per_s` is the drop-in call (row-major weights, sp_mlp_forward) in the one-launch-over-many-batches
    # timing mode; the other three combinations of weights and timing mode stand next to it.
    mlp = {k: extra.get(k, {}).get("rows_per_s") for k in ("mlp_leduc_16384", "mlp_leduc_16384_rowmajor",
                                                           "mlp_leduc_16384x64_one_launch",
                                                           "mlp_leduc_16384x64_one_launch_rowmajor")}
    line = {
        "metric": "GEMM TFLOP/s (% MFMA peak) at 4096^3 bf16; fused MLP fwd rows/sec",
        "value": None if head["wall_ms"] is None else round(flops / (head["wall_ms"] * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": head["wall_ms"], "event_ms_per_step": head.get("ms"),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "C = A.B^T, M=N=K=4096, A/B bf16 row-major N(0,1)/sqrt(K) (seed 2), f32 accumulate, "
                               "f32 output", "tile": head["tile"]},
        "roofline": head["roofline"], "cpu_baseline": cpu,
        "shader_clock_mhz": head.get("shader_clock_mhz"),
        "mlp_rows_per_s": mlp["mlp_leduc_16384x64_one_launch_rowmajor"],
        "mlp_rows_per_s_note": "the drop-in call sp_mlp_forward on the row-major weights the reference keeps, ONE launch over 64 "
                               "batches of 16384 rows (weights stay in registers across the batches); the packed-weights figures "
                               "assume weights packed once outside the timed region; the per-batch launch modes are in the detail",
        "mlp_rows_per_s_detail": {
            "row_major_weights_one_launch_over_64_batches": mlp["mlp_leduc_16384x64_one_launch_rowmajor"],
            "packed_weights_one_launch_over_64_batches": mlp["mlp_leduc_16384x64_one_launch"],
            "row_major_weights_one_launch_per_batch": mlp["mlp_leduc_16384_rowmajor"],
            "packed_weights_one_launch_per_batch": mlp["mlp_leduc_16384"]},
        "extra": extra, "device": info,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
