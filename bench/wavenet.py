"""benchmark config 4 as a benchmark workload: backward pass of the 30-block WaveNet-style stack,
2 waveforms x 16000 samples, driven through the library's network sequencer from a network file.  A backward pass
consumes state that only the forward pass rebuilds (the skip layers' cleared error buffers, the tanh(context)
buffer that the gated layer overwrites with its gradient), so every timed backward is preceded by an untimed
forward pass; the backward itself is timed with events on the launch stream."""
import json
import os
import time

import numpy as np

import synth as WD

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0


def flops_per_sample(nb, Q, R, K, C):
    block = 2 * (2 * R * 2 * R) * 2 + 2 * C * 2 * R + 4 * R * R + 4 * R * K  # cnn dX+dW (2 live taps), cond dW, out, skip 1x1
    return nb * block + 4 * K * K + 4 * K * Q + 2 * Q * R


def run(args, pkg):
    import torch

    import workloads as BW

    capi = pkg.capi
    nb, Q, R, K, C = 30, 1024, 64, 128, 80
    lengths = [16000, 16000]
    S, T = 2, 16000
    pat, onehot, ctx, target, N = WD.make(lengths, Q, C, upsample=80, seed=4)
    topology = pkg.specs.wavenet_network_doc(nb, Q, R, K, C, 1, 10)
    net = capi.Network(json.dumps(topology), S, T, mdn_config=[1, 0, Q, 0, 1, -1])
    # rows a dense layer's weight-gradient launch reads per sample: its input and its output errors
    dense_rows = [prev["size"] + cur["size"] for prev, cur in zip(topology["layers"], topology["layers"][1:])
                  if cur["type"].startswith("feedforward")]
    shapes = {L["name"]: L["weight_count"] for L in net.layers if L["weight_count"]}
    for k, w in WD.init_weights(shapes, seed=5).items():
        net.layer(k)["weights"].copy_(torch.from_numpy(w))
    ctx_d, pat_d = BW._dev(ctx), BW._dev(pat)
    net.set_context(ctx_d)
    net.load_sequences(pat_d, T, T, torch.zeros(N, dtype=torch.float32, device="cuda"), BW._dev(target))
    del onehot  # the feedback layer builds the teacher-forced one-hot input from the targets

    def timed_backward(n):
        total = 0.0
        for _ in range(n):
            net.forward()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            net.backward()
            e1.record()
            torch.cuda.synchronize()
            total += e0.elapsed_time(e1) * 1e-3
        return total / n

    timed_backward(args.warmup)
    sec = timed_backward(args.steps)
    net.forward()
    torch.cuda.synchronize()
    capi.profile_enable(True)
    net.backward()
    torch.cuda.synchronize()
    prof = capi.profile_read()
    capi.profile_enable(False)
    kernels = {k: {"launches": n, "avg_ms": ms / max(n, 1), "ms_per_step": ms} for k, (n, ms) in prof.items()}
    dom = max(kernels, key=lambda k: kernels[k]["ms_per_step"])
    step_flops = flops_per_sample(nb, Q, R, K, C) * N
    roof = {"bound": "hbm", "kernel": dom, "traffic": None, "peak": PEAK_HBM_GBS, "unit": "GB/s"}
    if dom == "wavenet_block_errors+cnn" and (R, K, N) == (64, 128, 32000):
        # two rocprofv3 --pmc runs (FETCH_SIZE x 2.00 by a copy of known size, WRITE_SIZE x 1.00) of this workload:
        # 104.6 MB read + 55.5 MB written per launch of wavenet_block_errors_kernel<64, 128, true>
        roof["traffic"] = 160.1e6
        roof["traffic_source"] = "profiles/wavenet_c4_backward_kernel_stats.md"
    if dom == "wavenet_block_errors+cnn":
        # one residual block's error path: reads the skip errors (K), what the later block handed on (R), the deltas of
        # the convolution above (2R, both taps from the same array), the gate pre-activations, the convolution's tanh
        # outputs and the conditioning tanh (2R each); writes the block's summed errors (R, which the earlier block's
        # launch reads where they stand), the convolution deltas and the conditioning gradient (2R each)
        nbytes = ((K + R + 4 * 2 * R) + (R + 2 * 2 * R)) * 4.0 * N
    elif dom == "gemm:cnn_dW":
        # per launch: read x (R) and the deltas (2R) for each of the two live taps, write nothing of size N
        nbytes = 2 * (R + 2 * R) * 4.0 * N
    elif dom == "gemm:cnn_prev_errors":
        nbytes = (2 * 2 * R + R) * 4.0 * N
    elif dom in ("gemm:dense_dW", "gemm:dense_prev_errors"):
        # average over the stack's dense layers (30 x 64->64, 30 x 64->128, the 1024->64 embedding, 128->128, 128->1024):
        # the weight gradient reads a layer's input and deltas, the error product reads the deltas and writes the
        # preceding layer's errors (the skip layer's step in its epilogue is not counted), over the launches made
        # (weight gradients: eight layers per launch)
        nbytes = sum(dense_rows) * 4.0 * N / kernels[dom]["launches"]
    else:
        nbytes = 155e3 * N / max(1, sum(v["launches"] for v in kernels.values()))
    roof["achieved"] = nbytes / (kernels[dom]["avg_ms"] * 1e-3) / 1e9
    roof["frac"] = roof["achieved"] / PEAK_HBM_GBS
    extra = {"roofline": roof, "kernels": kernels,
             "step_roofline": {"bound": "hbm", "achieved": 155e3 * N / sec / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                               "frac": 155e3 * N / sec / 1e9 / PEAK_HBM_GBS, "bytes_per_sample": 155e3,
                               "mfma_tflops": step_flops / sec / 1e12}}
    if not args.no_cpu:
        import oracle_models as OM  # the checker, only for this reported baseline

        # one block-sized slice of the same stack on the oracle: 2 blocks, 2 x 600 samples, scaled per sample and block
        nb_s, T_s = 2, 600
        p2, o2, c2, t2, N2 = WD.make([T_s, T_s], Q, C, upsample=80, seed=4)
        ref = OM.WaveNet(OM.OracleBackend(), nb_s, S, T_s, Q=Q, R=R, K=K, C=C, cnn_tanh=1)
        sh = {k: len(ref.buf[k]["W"]) for k in ref.weight_names()}
        for k, w in WD.init_weights(sh, seed=5).items():
            ref.buf[k]["W"][:] = w
        ref.set_inputs(p2, o2, c2, t2)
        ref.forward()
        t0 = time.perf_counter()
        ref.backward()
        dt = time.perf_counter() - t0
        # cost model: per-sample cost = a*blocks + b; measured with 2 blocks; the block-independent part (softmax
        # layers) is included once, so scaling the whole by 30/2 overstates the CPU's speed: say so
        extra["cpu_baseline"] = {"value": N2 / dt * nb_s / nb, "unit": "samples/s", "cores": 1, "kind": "port",
                                 "sample": "CPU oracle on the same topology with 2 of the 30 blocks and 2 x 600 samples "
                                           "(%.1f s), scaled by 2/30 per sample; host has %d cores" % (dt, os.cpu_count() or 0)}
    net.close()
    return BW._base(args, N / sec, "samples/s", sec,
                    "configs[3]: WaveNet-style stack backward, 30 blocks (dilations 1..512 x3), 64 residual / 128 skip "
                    "channels, 80-dim conditioning, 1024-way softmax, 2 x 16000 samples", extra)
