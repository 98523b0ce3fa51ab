#!/usr/bin/env python3
"""Benchmark of the backward hot path on one MI355X.

Workload: benchmark config 2, the acoustic model 382 -> 2 x feedforward_tanh 512 -> 2 x blstm 512
(256 cells per direction) -> feedforward_identity 187 -> sse, T = 600 frames, 10 parallel sequences
with lengths U{300..600}, fp32, synthetic seeded data, weights U(-0.08, 0.08).

A step is one full backward pass of the network over the resident fraction (all inputs, states and
weights already in HBM): per-fraction clearing of the stored output-gate deltas, SSE error, dense and
BLSTM backward including every weight gradient.  `value` is valid frames per second of that pass.
The forward pass that produces the states is run before the timed region (and timed separately as
`forward_backward_ms`).

Prints ONE JSON line.  Besides the contract fields it carries
  roofline      for the kernel family with the largest share of the step, measured live with HIP events
                on the launch stream (cnt_profile_enable) over a second run of the same K steps;
  cpu_baseline  the CPU oracle (a sequential restatement of the reference's host path, 1 core) timed on a
                bounded sample of the same network.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "bench"))   # the secondary workloads and the synthetic-data generators
sys.path.insert(0, os.path.join(ROOT, "oracle"))  # the CPU checker: imported only by the cpu_baseline legs

import numpy as np  # noqa: E402

# HBM bytes one launch of the backward recursion kernel moves on this workload (T=600, S=10, H=256, two directions),
# from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) scaled by a copy of known size; the figure and the command
# that made it are in the profile named here.  Algorithmic bytes of the same launch (T = 600): 123 MB.  None = not measured
# for the kernel this tree runs.
CHAIN_TRAFFIC_BYTES = 176.8e6  # (48 280 KiB x 2.00 fetched + 76 128 KiB written) per launch of lstm_backward_local<256, 8>
CHAIN_TRAFFIC_SOURCE = "profiles/acoustic_backward_hbm_traffic.md"
# The counters were read for this kernel, built from this source text (first 16 hex digits of the SHA-256 of
# csrc/lstm_local.hpp); when the file has changed since, the figure no longer describes the kernel that runs and the
# benchmark prints null for it.
CHAIN_TRAFFIC_KERNEL = "lstm_backward_local<256, 8>"
CHAIN_TRAFFIC_SOURCE_SHA16 = "1e7524efa6f2effe"

METRIC = "BLSTM backward frames/sec at 1 MI355X; % HBM/MFMA roofline vs host CPU"
PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0


def chain_traffic():
    """(bytes per launch, what they were measured on), or (None, why not) when the kernel's source has changed since."""
    import hashlib

    path = os.path.join(ROOT, "project-currennt-public_amd", "csrc", "lstm_local.hpp")
    try:
        with open(path, "rb") as f:
            now = hashlib.sha256(f.read()).hexdigest()[:16]
    except OSError:
        now = None
    measured_on = {"kernel": CHAIN_TRAFFIC_KERNEL, "source_sha16": CHAIN_TRAFFIC_SOURCE_SHA16, "profile": CHAIN_TRAFFIC_SOURCE}
    if now != CHAIN_TRAFFIC_SOURCE_SHA16:
        measured_on["stale"] = "csrc/lstm_local.hpp is now %s: the counters have not been read for this kernel" % now
        return None, measured_on
    return CHAIN_TRAFFIC_BYTES, measured_on


def make_fraction(seed, S, Tmax, Tlo, in_dim, out_dim, pin_longest=False):
    rng = np.random.default_rng(seed)
    lengths = [int(v) for v in rng.integers(Tlo, Tmax + 1, size=S)]
    if pin_longest:
        # the fraction is as long as the configuration says: the longest draw is made Tmax
        lengths[lengths.index(max(lengths))] = Tmax
    T = max(lengths)
    x = rng.standard_normal((T, S, in_dim)).astype(np.float32)
    tgt = rng.standard_normal((T, S, out_dim)).astype(np.float32)
    pat = np.zeros((T, S), dtype=np.int8)
    for s, n in enumerate(lengths):
        x[n:, s] = 0
        tgt[n:, s] = 0
        pat[:n, s] = 2
        pat[0, s] = 1
        pat[n - 1, s] = 3
    return lengths, T, x.reshape(-1), tgt.reshape(-1), pat.reshape(-1)


def backward_flops_per_slot(input_size, specs):
    """Algorithmic multiply-add flops of one backward pass per (t, s) slot."""
    fl, prev = 0.0, input_size
    for i, sp in enumerate(specs):
        t, D = sp["type"], sp["size"]
        if t.startswith("feedforward"):
            fl += 2.0 * prev * D * (1 if i == 0 else 2)  # dW always, dX unless it feeds the input layer
        elif t in ("lstm", "blstm"):
            nd = 2 if t == "blstm" else 1
            H = D // nd
            # recurrent 8H^2 + dW_int 8H^2 + dW_in 8HP + e_x 8HP per direction
            fl += nd * (16.0 * H * H + 16.0 * H * prev)
        prev = D
    return fl


def cpu_baseline(input_size, specs, S, seed, sample_T):
    """Times the oracle's backward on a short fraction of the same network (one core, sequential)."""
    import oracle_models as OM  # the checker, only for this reported baseline

    lengths, T, x, tgt, pat = make_fraction(seed, S, sample_T, max(1, sample_T // 2), input_size, specs[-1]["size"])
    weights = OM.init_weights(input_size, specs, seed + 1, 0.08)
    net = OM.OracleNetwork(input_size, specs, S, T, min(lengths), pat, weights)
    net.forward(x, tgt)
    t0 = time.perf_counter()
    net.backward()
    dt = time.perf_counter() - t0
    frames = sum(lengths)
    return {
        "value": frames / dt, "unit": "frames/s", "cores": 1, "kind": "port",
        "sample": "same network and weights distribution, one backward pass of a fraction with T=%d, S=%d "
                  "(%d valid frames, %.1f s); CPU oracle = sequential restatement of the reference's Thrust-host "
                  "path (naive k-ordered products, one loop per weight), g++ -O2, host has %d cores"
                  % (T, S, frames, dt, os.cpu_count() or 0),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--cpu-sample-T", type=int, default=160)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline leg")
    ap.add_argument("--workload", default="acoustic", choices=["acoustic", "lstm_c1", "mdn_c3", "dft_c5", "wavenet_c4", "opt_step", "nc_fraction"],
                    help="acoustic = benchmark configs[1] (the headline metric); the others are the remaining configs")
    ap.add_argument("--via-layer-calls", action="store_true",
                    help="also time the same backward pass through one C-ABI call per layer on one stream (the binding "
                         "a shell around the reference's Layer classes would use) and print it as `via_layer_calls`")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy (a kernel of known traffic, to scale rocprofv3's "
                         "FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path has no multi-GPU part); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from __graft_entry__ import load_package

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    pkg = load_package()
    capi = pkg.capi
    if args.calibrate_copy:
        a = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device="cuda")
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        del a, b
    if args.workload != "acoustic":
        import workloads

        print(json.dumps(workloads.run(args.workload, args, pkg)))
        return

    S, Tmax, seed = 10, 600, 20240
    input_size, specs = pkg.specs.acoustic_model_spec()
    lengths, T, x, tgt, pat = make_fraction(seed, S, Tmax, 300, input_size, 187, pin_longest=True)
    frames = sum(lengths)

    # the network file a user of the reference would write for this model, handed to the library's sequencer
    layers = [{"size": input_size, "name": "input", "type": "input"}]
    for i, sp in enumerate(specs):
        layers.append(dict(sp, name="%s_%d" % (sp["type"], i + 1)))
    net = capi.Network(json.dumps({"layers": layers}), S, T)
    # weights: seeded U(-0.08, 0.08), generated on the host with the same generator the parity tests use
    rng = np.random.default_rng(seed + 1)
    for L in net.layers:
        if L["weight_count"]:
            L["weights"].copy_(torch.from_numpy(rng.uniform(-0.08, 0.08, L["weight_count"]).astype(np.float32)))
    pat_d = torch.from_numpy(pat).cuda()
    net.load_sequences(pat_d, T, min(lengths), torch.from_numpy(x).cuda(), torch.from_numpy(tgt).cuda())
    net.forward()
    net.check()

    def step():
        net.load_sequences(pat_d, T, min(lengths))  # per-fraction clearing of the stored output-gate deltas
        net.backward()  # weight-gradient halves on the library's second stream, joined before it returns

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    net.check()
    ms_per_step = 1e3 * dt / args.steps
    value = frames * args.steps / dt

    # forward + backward, for information
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        net.load_sequences(pat_d, T, min(lengths))
        net.forward()
        net.backward()
    torch.cuda.synchronize()
    fb_ms = 1e3 * (time.perf_counter() - t0) / args.steps

    # per-kernel durations over the same K steps, HIP events on the launch stream
    capi.profile_enable(True)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    prof = capi.profile_read()
    capi.profile_enable(False)
    net.check()
    kernels = {k: {"launches": n, "avg_ms": ms / max(n, 1), "ms_per_step": ms / args.steps}
               for k, (n, ms) in prof.items()}
    dom = max(kernels, key=lambda k: kernels[k]["ms_per_step"])
    dom_avg_s = kernels[dom]["avg_ms"] * 1e-3

    H = 256
    slots = T * S
    if dom == "lstm_backward_chain":
        # one launch = both directions of one BLSTM layer over all T*S slots; the only dense work on the
        # recursion is the recurrent product, 8*H^2 flops per slot and direction
        flops = 2 * 8.0 * H * H * slots
        # What bounds a recursion of T dependent steps is not the matrix pipe but the hop every step ends with: the
        # library's probe measures one hop between two workgroups of an XCD with a step's arithmetic in between.
        def probe(**kw):
            # a diagnostic figure: a probe whose two workgroups do not meet must not cost the benchmark line
            try:
                return capi.probe_hop_latency(rounds=2000, **kw)
            except RuntimeError:
                return None

        hop_us = probe(same_xcd=True, with_compute=True)
        hop_bare_us = probe(same_xcd=True, with_compute=False)
        hop_far_us = probe(same_xcd=False, with_compute=False)

        def message(kb):
            try:
                return capi.probe_hop_message(kb, rounds=2000)
            except RuntimeError:
                return None
        us_per_step = 1e3 * kernels[dom]["avg_ms"] / T
        traffic, measured_on = chain_traffic()
        roof = {"bound": "mfma", "achieved": flops / dom_avg_s / 1e12, "peak": PEAK_FP32_MFMA_TFLOPS,
                "unit": "TFLOP/s", "traffic": traffic, "traffic_measured_on": measured_on,
                "kernel": dom,
                "us_per_step": us_per_step,
                "latency_floor_us_per_step": hop_us,
                "frac_of_latency_floor": hop_us / us_per_step if hop_us else None,
                "hop_us": {"same_xcd": hop_bare_us, "same_xcd_with_step_arithmetic": hop_us, "across_xcds": hop_far_us,
                           # what a workgroup receives per step: 4 KB today, 16 KB if partial pre-activations travelled
                           "message_4kb_same_xcd": message(4), "message_16kb_same_xcd": message(16)},
                "note": "latency-bound recursion: T sequential steps, each a 256x1024x%d product cut into (direction, "
                        "sequence group) jobs of 32 workgroups per XCD plus one exchange through that XCD's L2; `frac` is "
                        "against the fp32 MFMA peak as the metric asks, `frac_of_latency_floor` against T x (one measured "
                        "hop + a step's arithmetic), the bound that applies" % S}
    elif dom.startswith("gemm"):
        flops = backward_flops_per_slot(input_size, specs) * slots / max(1, len([k for k in kernels if k.startswith("gemm")]))
        roof = {"bound": "mfma", "achieved": flops / dom_avg_s / 1e12, "peak": PEAK_FP32_MFMA_TFLOPS,
                "unit": "TFLOP/s", "traffic": None, "kernel": dom}
    else:
        nbytes = 40.0 * H * slots
        roof = {"bound": "hbm", "achieved": nbytes / dom_avg_s / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "traffic": None, "kernel": dom}
    roof["frac"] = roof["achieved"] / roof["peak"]

    # useful work: the valid frames (padding slots do no useful work); the padded-slot figure is kept beside it
    step_flops = backward_flops_per_slot(input_size, specs) * frames
    step_flops_padded = backward_flops_per_slot(input_size, specs) * slots
    out = {
        "metric": METRIC, "value": value, "unit": "frames/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: acoustic model 382-512t-512t-blstm512-blstm512-187 + sse, full backward "
                               "pass, T=%d, S=%d, lengths U{300..600}, %d valid frames" % (T, S, frames),
                   "T": T, "parallel_sequences": S, "valid_frames": frames},
        "roofline": roof,
        "step_roofline": {"bound": "mfma", "achieved": step_flops / (ms_per_step * 1e-3) / 1e12,
                          "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                          "frac": step_flops / (ms_per_step * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS,
                          "flops_per_frame": backward_flops_per_slot(input_size, specs),
                          "counted": "valid frames (%d of %d slots)" % (frames, slots),
                          "frac_over_padded_slots": step_flops_padded / (ms_per_step * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS,
                          "note": "frac_over_padded_slots prices every slot, as the reference's schedule multiplies them; "
                                  "the library's weight gradients sum over the valid slots only, its other products "
                                  "over all slots"},
        "forward_backward_ms": fb_ms,
        "kernels": kernels,
    }
    net.close()
    if args.via_layer_calls:
        import layer_calls

        model = layer_calls.LayerCallModel(capi, input_size, specs, S, T, np.random.default_rng(seed + 1), 0.08)
        model.load_sequences(pat_d, T, min(lengths), torch.from_numpy(x).cuda(), torch.from_numpy(tgt).cuda())
        model.forward()
        model.check()

        def layer_step():
            model.load_sequences(pat_d, T, min(lengths))
            model.backward()

        for _ in range(args.warmup):
            layer_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            layer_step()
        torch.cuda.synchronize()
        dt2 = time.perf_counter() - t0
        model.check()
        model.close()
        out["via_layer_calls"] = {"value": frames * args.steps / dt2, "unit": "frames/s", "ms_per_step": 1e3 * dt2 / args.steps,
                                  "note": "same model and fraction, one C-ABI call per layer on one stream (no side streams)"}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(input_size, specs, S, seed, args.cpu_sample_T)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
