"""Secondary benchmark workloads (benchmark configs 1, 3, 4, 5), reached through `bench.py --workload ...`.
Each returns the same JSON fields as the headline workload: value in the config's unit, a roofline entry for
the dominant kernel (duration from the library's HIP-event hooks) and a cpu_baseline (the oracle, one core)."""
import os
import time

import numpy as np

from synth import make_pat_types

METRIC = "BLSTM backward frames/sec at 1 MI355X; % HBM/MFMA roofline vs host CPU"
PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0


def _timed(step, steps, warmup):
    import torch

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def _profile(capi, step, steps):
    import torch

    capi.profile_enable(True)
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    prof = capi.profile_read()
    capi.profile_enable(False)
    return {k: {"launches": n, "avg_ms": ms / max(n, 1), "ms_per_step": ms / steps} for k, (n, ms) in prof.items()}


def _base(args, value, unit, sec, workload, extra):
    out = {"metric": METRIC, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": 1e3 * sec, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
           "data": "synthetic", "config": {"workload": workload}}
    out.update(extra)
    return out


def _dev(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def lstm_c1(args, pkg):
    import torch

    capi = pkg.capi
    P, H, S, lengths = 382, 256, 4, [200, 200, 200, 150]
    T, N = 200, 800
    rng = np.random.default_rng(1)
    nW = capi.lib().cnt_lstm_weight_count(P, H, 0)
    W = rng.uniform(-0.1, 0.1, nW).astype(np.float32)
    x = rng.standard_normal((T, S, P)).astype(np.float32)
    err = (0.1 * rng.standard_normal((T, S, H))).astype(np.float32)
    x[150:, 3] = 0
    err[150:, 3] = 0
    pat = make_pat_types(lengths, T)
    layer = capi.Lstm(P, H, False, S, T, 1.0)
    Wd, xd, pd = _dev(W), _dev(x.reshape(-1)), _dev(pat)
    out = torch.zeros(H * N, device="cuda")
    ex = torch.zeros(P * N, device="cuda")
    dW = torch.zeros(nW, device="cuda")
    err0 = _dev(err.reshape(-1))
    errd = err0.clone()
    layer.load_sequences(pd, T, 150)
    layer.forward(Wd, xd, out)

    def step():
        errd.copy_(err0)  # the unidirectional backward adds the recurrent terms in place
        layer.load_sequences(pd, T, 150)
        layer.backward(Wd, xd, out, errd, ex, dW)

    sec = _timed(step, args.steps, args.warmup)
    layer.check()
    kernels = _profile(capi, step, args.steps)
    frames = sum(lengths)
    dom = "lstm_backward_chain"
    flops = 8.0 * H * H * N
    ach = flops / (kernels[dom]["avg_ms"] * 1e-3) / 1e12
    us_per_step = kernels[dom]["avg_ms"] * 1e3 / T
    hop_us = capi.probe_hop_latency(same_xcd=True, with_compute=True, rounds=2000)
    roof = {"bound": "mfma", "achieved": ach, "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s", "frac": ach / PEAK_FP32_MFMA_TFLOPS,
            # two rocprofv3 --pmc runs of this workload (FETCH_SIZE x 2.00 by a copy of known size, WRITE_SIZE x 1.00):
            # 12.2 MB read + 7.0 MB written per launch of lstm_backward_local<256, 8>; algorithmic 12.5 MB
            "traffic": 19.2e6, "traffic_source": "profiles/lstm_c1_backward_kernel_stats.md",
            "kernel": dom, "us_per_step": us_per_step, "latency_floor_us_per_step": hop_us,
            "frac_of_latency_floor": hop_us / us_per_step,
            "note": "latency-bound recursion (T sequential steps, one job of four sequences on one XCD): `frac` is against the "
                    "fp32 MFMA peak, `frac_of_latency_floor` against one measured hop inside an XCD plus a step's arithmetic"}
    extra = {"roofline": roof, "kernels": kernels}
    if not args.no_cpu:
        import oracle_lib as O  # the checker, only for this reported baseline

        desc = O.LstmDesc(P, H, 0, S, T, 150, 1.0)
        fw = O.LstmState(H, N)
        o = np.zeros(H * N, dtype=np.float32)
        O.lstm_forward(desc, W, pat, x.reshape(-1), fw, None, o)
        exo, dWo = np.zeros(P * N, dtype=np.float32), np.zeros_like(W)
        t0 = time.perf_counter()
        O.lstm_backward(desc, W, pat, x.reshape(-1), err.reshape(-1), fw, None, exo, dWo)
        dt = time.perf_counter() - t0
        extra["cpu_baseline"] = {"value": frames / dt, "unit": "frames/s", "cores": 1, "kind": "port",
                                 "sample": "the full config-1 backward once (%.1f s), CPU oracle, host has %d cores" % (dt, os.cpu_count() or 0)}
    layer.close()
    return _base(args, frames / sec, "frames/s", sec,
                 "configs[0]: unidirectional LSTM P=382 H=256 T=200 S=4 (one sequence of 150), full BPTT backward", extra)


def mdn_c3(args, pkg):
    import torch

    capi = pkg.capi
    M, D, S, T = 16, 60, 10, 600
    F, Lp = S * T, 16 + 2 * 16 * 60
    rng = np.random.default_rng(3)
    x = rng.standard_normal((F, Lp)).astype(np.float32)
    x[:, M + M * D:] *= 0.5
    tgt = rng.standard_normal((F, D)).astype(np.float32)
    pat = make_pat_types([T] * S, T)
    layer = capi.Mdn(Lp, D, S, T, [1, 0, Lp, 0, D, M])
    pd, xd, td = _dev(pat), _dev(x.reshape(-1)), _dev(tgt.reshape(-1))
    res = torch.zeros(1, device="cuda")
    err = torch.zeros(F * Lp, device="cuda")
    layer.load_sequences(pd, T)
    layer.forward(xd)
    layer.calculate_error(td, res)

    def step():
        # the gradient needs the posteriors of the error pass (MDNUnit.cu:6037-6193 before :6222), so a step is both:
        # one call, one pass over the parameters
        layer.error_backward(td, res, err)

    def step_two_calls():
        layer.calculate_error(td, res)
        layer.backward(td, err)

    sec = _timed(step, args.steps, args.warmup)
    kernels = _profile(capi, step, args.steps)
    sec_two = _timed(step_two_calls, args.steps, args.warmup)
    kernels.update(_profile(capi, step_two_calls, args.steps))
    dom = "mdn_mixture_error_backward"
    # weights, means, deviations and targets in; Lp errors and the M + 1 log-likelihood terms out
    nbytes = F * (Lp + D + Lp + M + 1) * 4
    ach = nbytes / (kernels[dom]["avg_ms"] * 1e-3) / 1e9
    # traffic: two rocprofv3 --pmc runs of this workload (FETCH_SIZE 23 975 KiB x 2.00 by a copy of known size, WRITE_SIZE
    # 54 442 KiB x 1.00) for the benchmark size; other sizes have not been read
    roof = {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": ach / PEAK_HBM_GBS,
            "traffic": 104.8e6 if (F, M, D) == (6000, 16, 60) else None,
            "traffic_source": "profiles/mdn_c3_backward_kernel_stats.md", "kernel": dom}

    def full():
        layer.forward(xd)
        layer.error_backward(td, res, err)

    sec_full = _timed(full, args.steps, 1)
    extra = {"roofline": roof, "kernels": kernels, "forward_error_backward_ms": 1e3 * sec_full,
             "error_then_backward_two_calls_ms": 1e3 * sec_two}
    if not args.no_cpu:
        import oracle_lib as O  # the checker, only for this reported baseline

        para = np.zeros(F * M * (1 + 2 * D), dtype=np.float32)
        tmp = np.zeros(F * M + F, dtype=np.float32)
        eo = np.zeros(F * Lp, dtype=np.float32)
        O.mdn_mixture_forward(F, Lp, 0, M, D, 0.0, pat, x.reshape(-1), para)
        O.mdn_mixture_error(F, D, 0, M, D, pat, tgt.reshape(-1), para, tmp)
        t0 = time.perf_counter()
        for _ in range(20):
            O.mdn_mixture_backward(F, Lp, D, 0, 0, M, D, 0.0, pat, tgt.reshape(-1), para, tmp, eo)
        dt = (time.perf_counter() - t0) / 20
        extra["cpu_baseline"] = {"value": F / dt, "unit": "frames/s", "cores": 1, "kind": "port",
                                 "sample": "the full config-3 gradient, 20 repetitions (%.2f s each), CPU oracle, host has %d cores" % (dt, os.cpu_count() or 0)}
    layer.close()
    return _base(args, F / sec, "frames/s", sec,
                 "configs[2]: mixture density layer backward, 16 mixtures x 60 dims, T=600 S=10 (6000 frames)", extra)


def dft_c5(args, pkg):
    import torch

    capi = pkg.capi
    res = [(512, 512, 80), (128, 128, 40), (2048, 2048, 640)]
    W, n = 8, 16000
    rng = np.random.default_rng(5)
    src = (0.3 * rng.standard_normal((W, n))).astype(np.float32)
    tgt = (0.3 * rng.standard_normal((W, n))).astype(np.float32)
    layer = capi.Dft(res, n, W)
    sd, td = _dev(src.reshape(-1)), _dev(tgt.reshape(-1))
    errs = torch.zeros(W * 3, device="cuda")
    grad = torch.zeros(W * n, device="cuda")

    def step():
        layer.forward([n] * W, sd, td, errs)
        layer.backward(grad)

    sec = _timed(step, args.steps, args.warmup)
    kernels = _profile(capi, step, args.steps)
    dom = "dft_loss"
    nbytes = 12.0 * W * n  # per launch (all three resolutions in it): read source + target once, write the gradient once
    ach = nbytes / (kernels[dom]["avg_ms"] * 1e-3) / 1e9
    # traffic: two rocprofv3 --pmc runs of this workload (FETCH_SIZE x 2.00 by a copy of known size, WRITE_SIZE x 1.00):
    # dft_loss_kernel 6.3 MB read (every sample is part of four frames per resolution) + 6.3 MB written (overlap-add)
    roof = {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": ach / PEAK_HBM_GBS,
            "traffic": 12.6e6 if (W, n) == (8, 16000) else None, "traffic_source": "profiles/dft_c5_backward_kernel_stats.md",
            "kernel": dom, "note": "1.5 MB of samples and gradients, 0.17 GFLOP: launch- and latency-bound, far from either roof"}
    extra = {"roofline": roof, "kernels": kernels}
    if not args.no_cpu:
        import oracle_lib as O  # the checker, only for this reported baseline

        g = np.zeros(n, dtype=np.float32)
        t0 = time.perf_counter()
        for (N, Nw, Hs) in res:
            O.dft_logamp_loss(N, Nw, Hs, 0, n, n, 1.0, 1e-5, src[0].copy(), tgt[0].copy(), g)
        dt = time.perf_counter() - t0
        extra["cpu_baseline"] = {"value": n / dt, "unit": "samples/s", "cores": 1, "kind": "port",
                                 "sample": "one of the 8 waveforms, all three resolutions (%.2f s); the reference has no host FFT, "
                                           "the oracle's own double-precision radix-2 FFT is used; host has %d cores" % (dt, os.cpu_count() or 0)}
    layer.close()
    return _base(args, W * n / sec, "samples/s", sec,
                 "configs[4]: DFT multi-resolution log-amplitude loss, forward (loss + gradient) and backward, 8 x 16000 samples", extra)


def opt_step(args, pkg):
    """Adam step (copy + adjust + update in one pass) over the acoustic model's 3.7 M weights: the network
    sequencer keeps all weights in one array, so the step is one launch."""
    import json

    import torch

    capi = pkg.capi
    input_size, specs = pkg.specs.acoustic_model_spec()
    layers = [{"size": input_size, "name": "input", "type": "input"}]
    layers += [dict(sp, name="l%d" % i) for i, sp in enumerate(specs)]
    net = capi.Network(json.dumps({"layers": layers}), 10, 16)
    net.randomize(5, 0.08)
    net.updates.copy_(torch.randn(net.n_weights, device="cuda"))
    sizes = [L["weight_count"] for L in net.layers if L["weight_count"]]
    assert sizes == [382 * 512 + 512, 512 * 512 + 512, 1576448, 1576448, 512 * 187 + 187]

    def step():
        net.update(capi.OPT_ADAM, 1e-4, 0.0, 4904.0)

    sec = _timed(step, args.steps, args.warmup)
    kernels = _profile(capi, step, args.steps)
    total = sum(sizes)
    nbytes = total * 40.0  # per weight: read g, m, v, delta, w; write cur, m, v, delta, w
    ach = nbytes / (kernels["opt_step"]["ms_per_step"] * 1e-3) / 1e9
    roof = {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": ach / PEAK_HBM_GBS,
            # two rocprofv3 --pmc runs of this workload: 74.2 MB fetched by the L2s + 74.2 MB written per launch
            "traffic": 148.4e6, "traffic_source": "profiles/opt_step_kernel_stats.md", "kernel": "opt_step",
            "note": "one launch over all 3.7 M weights; 40 B per weight = 148 MB per step, which repeated steps "
                    "find in the 256 MB last-level cache: the figure is not a pure HBM rate"}
    extra = {"roofline": roof, "kernels": kernels}
    if not args.no_cpu:
        import oracle_lib as O  # the checker, only for this reported baseline

        hw = [np.zeros(n, np.float32) for n in sizes]
        t0 = time.perf_counter()
        reps = 5
        for _ in range(reps):
            for n, w in zip(sizes, hw):
                g = np.ones(n, np.float32); cur = np.empty(n, np.float32)
                O.opt_accumulate(g, cur, False)
                O.opt_adjust_gradient(5, cur, np.zeros(2 * n, np.float32), None, 4904.0, 0.9, 0.999)
                O.opt_update_weights(w, cur, np.zeros(n, np.float32), None, 1e-4, 0.0)
        dt = (time.perf_counter() - t0) / reps
        extra["cpu_baseline"] = {"value": total / dt, "unit": "weights/s", "cores": 1, "kind": "port",
                                 "sample": "the same 3.7 M weights, %d repetitions, CPU oracle (three passes as in the reference)" % reps}
    return _base(args, total / sec, "weights/s", sec,
                 "optimizer step: Adam weight update of the acoustic model (3.7 M weights in 5 layers), one fused pass over the "
                 "sequencer's weight array", extra)


def nc_fraction(args, pkg):
    """Host-side: build the C2-shaped fraction (10 sequences of 300..600 frames, 382 inputs, 187 targets) from a
    .nc file.  No kernel runs; the figure is frames per second of the reader + interleaver on one host core."""
    import importlib.util
    import tempfile

    from scipy.io import netcdf_file

    capi = pkg.capi
    rng = np.random.default_rng(9)
    lengths = [int(v) for v in rng.integers(300, 601, 10)]
    total, P, Q, S = sum(lengths), 382, 187, 10
    tmp = tempfile.mkdtemp(prefix="cnt_nc_")
    path = os.path.join(tmp, "c2.nc")
    f = netcdf_file(path, "w", version=2)
    for name, n in (("numSeqs", S), ("numTimesteps", total), ("inputPattSize", P), ("targetPattSize", Q), ("maxSeqTagLength", 8)):
        f.createDimension(name, n)
    tags = f.createVariable("seqTags", "c", ("numSeqs", "maxSeqTagLength"))
    for i in range(S):
        tags[i] = np.frombuffer(("u%02d" % i).encode().ljust(8, b"\0"), dtype="S1")
    f.createVariable("seqLengths", "i", ("numSeqs",))[:] = np.asarray(lengths, np.int32)
    f.createVariable("inputs", "f", ("numTimesteps", "inputPattSize"))[:] = rng.standard_normal((total, P)).astype(np.float32)
    f.createVariable("targetPatterns", "f", ("numTimesteps", "targetPattSize"))[:] = rng.standard_normal((total, Q)).astype(np.float32)
    f.close()
    ds = capi.Dataset(path, S, True, 0, 1.0)

    def step():
        ds.fraction(0)

    for _ in range(args.warmup):
        step()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    sec = (time.perf_counter() - t0) / args.steps
    nbytes = total * (P + Q) * 4.0
    extra = {"roofline": {"bound": "hbm", "achieved": nbytes / sec / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                          "frac": nbytes / sec / 1e9 / PEAK_HBM_GBS, "traffic": None, "kernel": "none (host code)",
                          "note": "host-side reader: the figure is file bytes delivered per second by one CPU core; the "
                                  "HBM peak is listed only because the field is mandatory"}}
    if not args.no_cpu:
        import oracle_lib as O  # the checker, only for this reported baseline

        spec = importlib.util.spec_from_file_location("nc_fraction", os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "nc_fraction.py"))
        NF = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(NF)
        segs = NF.segments(path)
        t0 = time.perf_counter()
        NF.make_fraction(path, segs, 0, S)
        dt = time.perf_counter() - t0
        extra["cpu_baseline"] = {"value": total / dt, "unit": "frames/s", "cores": 1, "kind": "port",
                                 "sample": "the same fraction once, numpy oracle with scipy's NetCDF reader (%.2f s)" % dt}
    ds.close()
    os.remove(path)
    os.rmdir(tmp)
    return _base(args, total / sec, "frames/s", sec,
                 "next row f2: one C2-shaped fraction (%d frames, 382 inputs + 187 targets, S=10) from a 64-bit-offset .nc file, host code" % total,
                 extra)


def run(name, args, pkg):
    if name == "wavenet_c4":
        import wavenet

        return wavenet.run(args, pkg)
    return {"lstm_c1": lstm_c1, "mdn_c3": mdn_c3, "dft_c5": dft_c5, "opt_step": opt_step, "nc_fraction": nc_fraction}[name](args, pkg)
