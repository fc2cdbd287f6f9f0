#!/usr/bin/env python3
"""Benchmark of the MAM fully-connected hot path on one MI355X.

One "step" = one pass of the hot path over one synthetic batch of the headline configuration
(MAM FullyConnected fp32, batch 256, in = out = 4096): exact forward with argmax/argmin, backward
(grad_x, grad_W), and selection-count accumulation, launched back to back on one stream through
the C ABI of libmam_hip.so with all inputs already resident in HBM.

Prints ONE JSON line.  `value` is N*K*M / t_step in GOPS (one op = one multiply-max-min triple).
`roofline` describes the dominant kernel (the forward, FP32-VALU bound: 3 fp32 ops per triple
against 256 CUs x 128 lanes x 2.4 GHz = 78.6 T fp32-op/s, i.e. the 157.3 TFLOP/s vector peak
without the FMA factor that a (max, min, x) semiring cannot use).  `roofline_backward` gives the
backward's algorithmic bytes over its time against 8 TB/s.  `cpu_baseline` is the pure-PyTorch
restatement of the reference's CPU path (oracle/torch_port.py) timed on a bounded row sample.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

N, K, M = 256, 4096, 4096
VALU_PEAK_TFLOPS = 78.65      # 256 CU x 4 SIMD x 16 lanes x 2 (packed width) x 2.4 GHz, no FMA x2
VECTOR_FP32_PEAK_TFLOPS = 157.3
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch from the FETCH_SIZE / WRITE_SIZE counters, each scaled by what the same
# counter reads for the plain 64 MiB copy below (profiles/hbm_traffic_headline_n256_k4096_m4096.md)
FORWARD_TRAFFIC_BYTES = {"mam_fwd_kernel": 141.1e6, "mam_fwd_merge_kernel": 167.7e6}
BACKWARD_TRAFFIC_BYTES = {"mam_bwd_x_kernel": 25.2e6, "mam_bwd_w_vec_kernel": 103.4e6}


def make_inputs(torch, dev):
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(N, K, generator=gen)
    w = (torch.rand(M, K, generator=gen) * 2 - 1) / 64.0   # weight (out, in) ~ U(-1/64, 1/64)
    g = torch.randn(N, M, generator=gen)
    return x, w, g


def cpu_baseline(torch, x, w, g, budget_s):
    """Times forward + backward of the pure-PyTorch port on the first `rows` batch rows."""
    from oracle import torch_port

    b = w.T.contiguous()
    rows = 2
    t0 = time.perf_counter()
    y, amax, amin = torch_port.forward(x[:rows], b)
    torch_port.backward(x[:rows], b, g[:rows], amax, amin)
    per_row = (time.perf_counter() - t0) / rows
    rows = int(max(2, min(N, budget_s / max(per_row, 1e-6))))
    t0 = time.perf_counter()
    y, amax, amin = torch_port.forward(x[:rows], b)
    torch_port.backward(x[:rows], b, g[:rows], amax, amin)
    dt = time.perf_counter() - t0
    return {
        "value": round(rows * K * M / dt / 1e9, 4),
        "unit": "GOPS",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": "forward+backward of oracle/torch_port.py on the first %d of %d batch rows "
                  "(%.1f s); rows are independent, so GOPS does not depend on the row count" % (rows, N, dt),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=300,
                    help="untimed steps; the GPU clock needs ~100 launches to ramp up")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU baseline budget; 0 skips it")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the MAM hot path has no multi-GPU part in this build "
              "(--gpus %d refused)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch

    from mamtorch_amd import capi

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the MAM operators have no CPU path)", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    lib = capi.lib()
    x_cpu, w_cpu, g_cpu = make_inputs(torch, dev)
    x, w, g = x_cpu.to(dev), w_cpu.to(dev), g_cpu.to(dev)

    c = torch.empty((N, M), dtype=torch.float32, device=dev)
    amax = torch.empty((N, M), dtype=torch.int32, device=dev)
    amin = torch.empty((N, M), dtype=torch.int32, device=dev)
    xg = torch.empty((N, K), dtype=torch.float32, device=dev)
    wg = torch.empty((M, K), dtype=torch.float32, device=dev)
    max_count = torch.zeros((M, K), dtype=torch.int32, device=dev)
    min_count = torch.zeros((M, K), dtype=torch.int32, device=dev)
    ws_bytes = lib.mam_fc_forward_workspace(N, K, M)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    wsel = torch.empty((2, N, M), dtype=torch.float32, device=dev)   # selected weights, forward -> backward

    stream = torch.cuda.current_stream(dev)
    sp = ctypes.c_void_p(stream.cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())

    def forward():
        rc = lib.mam_fc_forward(P(x), K, P(w), K, capi.W_MK, None, P(c), P(amax), P(amin), P(wsel),
                                N, K, M, P(ws), ws_bytes, sp)
        assert rc == 0, lib.mam_last_error()

    def backward():
        rc = lib.mam_fc_backward(P(x), K, P(w), K, capi.W_MK, P(g), P(amax), P(amin), P(wsel), P(xg),
                                 P(wg), N, K, M, sp)
        assert rc == 0, lib.mam_last_error()

    def count():
        rc = lib.mam_selection_count(P(amax), P(amin), P(max_count), P(min_count), N, M, K,
                                     capi.COUNT_HITS, sp)
        assert rc == 0, lib.mam_last_error()

    # one plain 64 MiB copy kernel: the known-size reference that scales the profiler's
    # FETCH_SIZE / WRITE_SIZE counters when traffic is measured
    calibration_copy = max_count.clone()
    del calibration_copy

    for _ in range(args.warmup):
        forward(); backward(); count()
    torch.cuda.synchronize()

    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(args.steps):
        ev[s][0].record(stream)
        forward()
        ev[s][1].record(stream)
        backward()
        ev[s][2].record(stream)
        count()
        ev[s][3].record(stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()

    ms_step = (t1 - t0) * 1e3 / args.steps
    fwd_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / args.steps
    bwd_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / args.steps
    cnt_ms = sum(e[2].elapsed_time(e[3]) for e in ev) / args.steps

    triples = N * K * M
    fwd_tflops = 3.0 * triples / (fwd_ms * 1e-3) / 1e12
    bwd_bytes = 4 * (N * K + N * M + 2 * N * M + 2 * N * M + N * K + K * M)
    bwd_gbs = bwd_bytes / (bwd_ms * 1e-3) / 1e9

    out = {
        "metric": "MAM FC fwd+bwd GOPS @4096x4096 b256 fp32; % FP32 VALU peak; bwd HBM GB/s",
        "value": round(triples / (ms_step * 1e-3) / 1e9, 2),
        "unit": "GOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "MAM FullyConnected fp32 batch 256 in 4096 out 4096: exact forward with "
                        "argmax/argmin + backward (grad_x, grad_W) + selection-count accumulation; "
                        "x~N(0,1), W~U(-1/64,1/64), grad_out~N(0,1), seed 0; weight in (out,in) layout",
            "N": N, "K": K, "M": M,
        },
        "phases_ms": {"forward": round(fwd_ms, 5), "backward": round(bwd_ms, 5),
                      "selection_count": round(cnt_ms, 5)},
        "forward_gops": round(triples / (fwd_ms * 1e-3) / 1e9, 2),
        "fwd_bwd_gops": round(triples / ((fwd_ms + bwd_ms) * 1e-3) / 1e9, 2),
        "fwd_bwd_valu_frac": round(3.0 * triples / ((fwd_ms + bwd_ms) * 1e-3) / 1e12 / VALU_PEAK_TFLOPS, 4),
        "roofline": {
            "kernel": "mam_fwd_kernel<MK,args> + mam_fwd_merge_kernel (one mam_fc_forward call)",
            "bound": "valu",
            "achieved": round(fwd_tflops, 3),
            "peak": VALU_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(fwd_tflops / VALU_PEAK_TFLOPS, 4),
            "frac_of_vector_fp32_157.3": round(fwd_tflops / VECTOR_FP32_PEAK_TFLOPS, 4),
            "traffic": sum(FORWARD_TRAFFIC_BYTES.values()),
            "traffic_by_kernel": FORWARD_TRAFFIC_BYTES,
            "algorithmic_bytes": 4 * (N * K + K * M + 4 * N * M),
        },
        "roofline_backward": {
            "kernel": "mam_bwd_x_kernel + mam_bwd_w_vec_kernel",
            "bound": "hbm",
            "achieved": round(bwd_gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(bwd_gbs / HBM_PEAK_GBS, 4),
            "traffic": sum(BACKWARD_TRAFFIC_BYTES.values()),
            "traffic_by_kernel": BACKWARD_TRAFFIC_BYTES,
            "algorithmic_bytes": bwd_bytes,
        },
    }
    if args.cpu_seconds > 0:
        out["cpu_baseline"] = cpu_baseline(torch, x_cpu, w_cpu, g_cpu, args.cpu_seconds)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
