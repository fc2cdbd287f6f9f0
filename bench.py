#!/usr/bin/env python3
"""Benchmark of the MAM fully-connected hot path on one MI355X.

Default workload ("headline"): one "step" = one pass of the hot path over one synthetic batch of
MAM FullyConnected fp32, batch 256, in = out = 4096: exact forward with argmax/argmin, backward
(grad_x, grad_W), and selection-count accumulation (true hit counts), launched back to back on one
stream through the C ABI of libmam_hip.so with all inputs already resident in HBM.

Prints ONE JSON line.  `value` is (multiply-max-min triples per step) / t_step in GOPS.
`roofline` describes the dominant kernel: for the dense workloads the forward, FP32-VALU bound
(3 fp32 ops per triple against 256 CUs x 128 lanes x 2.4 GHz = 78.6 T fp32-op/s, i.e. the
157.3 TFLOP/s vector peak without the FMA factor that a (max, min, x) semiring cannot use); for
the CSR-sparse workloads the forward against HBM bandwidth.  `roofline_backward` gives the
backward's algorithmic bytes over its time against 8 TB/s.  `cpu_baseline` is the pure-PyTorch
restatement of the reference's CPU path (oracle/torch_port.py) timed on a bounded row sample.

Other workloads (`--workload`), same JSON layout, used for the tables in the design notes:
  vit_mlp            12608 rows through MAM FC 768->3072 and MAM FC 3072->768, forward + backward
  inference_m{1024,4096,16384}   batch 16384, in 4096, forward with indices only
  config1            batch 64, 784 -> 256: forward + backward + selection count (launch-latency bound)
  values_headline    headline shape, values-only forward
  sparse_d{10,03,01} 4096x4096 weight pruned to 10 % / 3 % / 1 %, batch 256, CSR forward + backward
  spmm_d{30,10,01}   sum-of-products SpMM (cusparsemm): 4096x4096 CSR with 30 % / 10 % / 1 % stored, times a
                     dense 4096x4096; one op = one multiply-add; torch.sparse.mm timed beside it
  spmm_sweep         the reference's sparse benchmark grid: sizes 128..4096 x sparse rates 0.7..0.999 x {COO, CSR}
  prune_csr          magnitude pruning of a 4096x4096 weight to 10 % and its compaction to CSR (row offsets +
                     fill); one op = one weight examined; Tensor.to_sparse_csr of the masked weight timed beside it
  module_headline    the path a user of the reference runs, at the headline shape: mamtorch.nn.FullyConnected(4096,
                     4096, store_args=True) forward, autograd backward and update_selection_count(); the same
                     step through the C ABI (pre-allocated outputs) is timed beside it in the same run
  module_vit_mlp     the same for the two layers of the ViT MLP block (12608 rows, 768 -> 3072 -> 768), no counting
  reference_script   the shape and the operator calls of the reference's own timing loop (test/test.py:186-323):
                     a (128, 2048) x b (2048, 4096) in the reference's (in, out) layout through torch.ops:
                     v1 fullyconnected, v4 fullyconnected, v4 fullyconnected_fast, v4 fullyconnected_backward with
                     random indices, torch.matmul beside them; a step = the four MAM operator calls
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Published MI355X peaks.  The vector FP32 figure (157.3 TFLOP/s) is 256 CUs x 128 fp32 lane-operations per
# clock x 2.4 GHz with a fused multiply-add counted as two; a (max, min, x) semiring has no fused form, so
# its yardstick counts one operation per lane and clock: 78.65 T fp32-op/s.
VALU_PEAK_TFLOPS = 78.65
VECTOR_FP32_PEAK_TFLOPS = 157.3
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch at the headline shape.  These are CONSTANTS copied from the committed counter
# summary named below (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, of this same command, each scaled by
# what the same counter reads for the plain 64 MiB copy made before the warm-up); they are not measured
# by the run that prints them.
TRAFFIC_PROFILE = "profiles/hbm_traffic_headline_n256_k4096_m4096.md"
FORWARD_TRAFFIC_BYTES = {"mam_fwd_sx_kernel": 136.2e6, "mam_fwd_merge_kernel": 141.4e6}
BACKWARD_TRAFFIC_BYTES = {"mam_bwd_x_kernel": 25.3e6, "mam_bwd_w_vec_kernel": 91.1e6}
SELCOUNT_TRAFFIC_BYTES = {"selcount_kernel": 166.4e6}
RAMP_MIN_CALLS = 300          # untimed phase calls before the counted warm-up: the GPU clock ramps over them
RAMP_MIN_SECONDS = 0.3
RAMP_MAX_SECONDS = 3.0

WORKLOADS = ("headline", "config1", "values_headline", "vit_mlp", "inference_m1024", "inference_m4096",
             "inference_m16384", "sparse_d10", "sparse_d03", "sparse_d01", "spmm_d30", "spmm_d10", "spmm_d01", "prune_csr",
             "reference_script", "module_headline", "module_vit_mlp", "spmm_sweep")


class Layer:
    """One dense MAM layer's buffers and its C-ABI calls on the current stream."""

    def __init__(self, torch, capi, lib, dev, x, w, g, want_backward, want_count, values_only=False):
        self.lib, self.capi = lib, capi
        self.N, self.K = x.shape
        self.M = w.shape[0]
        N, K, M = self.N, self.K, self.M
        self.x, self.w, self.g = x.to(dev), w.to(dev), None if g is None else g.to(dev)
        self.values_only = values_only
        self.c = torch.empty((N, M), dtype=torch.float32, device=dev)
        if not values_only:
            self.amax = torch.empty((N, M), dtype=torch.int32, device=dev)
            self.amin = torch.empty((N, M), dtype=torch.int32, device=dev)
        if want_backward:
            self.xg = torch.empty((N, K), dtype=torch.float32, device=dev)
            self.wg = torch.empty((M, K), dtype=torch.float32, device=dev)
            # selected weights and inputs, forward -> backward
            self.wsel = torch.empty((2, N, M), dtype=torch.float32, device=dev)
            self.xsel = torch.empty((2, N, M), dtype=torch.float32, device=dev)
        else:
            self.wsel = self.xsel = None
        if want_count:
            self.max_count = torch.zeros((M, K), dtype=torch.int32, device=dev)
            self.min_count = torch.zeros((M, K), dtype=torch.int32, device=dev)
        # what the operators and capi bring: the required bytes plus the optional room the library can use
        self.ws_bytes = lib.mam_fc_forward_workspace_for(N, K, M, capi.W_MK, 0 if values_only else 1)
        self.ws = torch.empty(max(self.ws_bytes, 1), dtype=torch.uint8, device=dev)
        self.torch, self.dev = torch, dev

    @staticmethod
    def _p(t):
        return None if t is None else ctypes.c_void_p(t.data_ptr())

    @property
    def sp(self):
        # the stream that is current at the call (the capture stream while a graph is recorded)
        return ctypes.c_void_p(self.torch.cuda.current_stream(self.dev).cuda_stream)

    def forward(self):
        P, N, K, M = self._p, self.N, self.K, self.M
        if self.values_only:
            rc = self.lib.mam_fc_forward_values(P(self.x), K, P(self.w), K, self.capi.W_MK, None, P(self.c),
                                                N, K, M, P(self.ws), self.ws_bytes, self.sp)
        else:
            rc = self.lib.mam_fc_forward(P(self.x), K, P(self.w), K, self.capi.W_MK, None, P(self.c),
                                         P(self.amax), P(self.amin), P(self.wsel), P(self.xsel), N, K, M, P(self.ws),
                                         self.ws_bytes, self.sp)
        assert rc == 0, self.lib.mam_last_error()

    def backward(self):
        P, N, K, M = self._p, self.N, self.K, self.M
        rc = self.lib.mam_fc_backward(P(self.x), K, P(self.w), K, self.capi.W_MK, P(self.g), P(self.amax),
                                      P(self.amin), P(self.wsel), P(self.xsel), P(self.xg), P(self.wg), N, K, M,
                                      self.sp)
        assert rc == 0, self.lib.mam_last_error()

    def count(self):
        P = self._p
        rc = self.lib.mam_selection_count(P(self.amax), P(self.amin), P(self.max_count), P(self.min_count),
                                          self.N, self.M, self.K, self.capi.COUNT_HITS, self.sp)
        assert rc == 0, self.lib.mam_last_error()

    def backward_count(self):
        P, N, K, M = self._p, self.N, self.K, self.M
        rc = self.lib.mam_fc_backward_count(P(self.x), K, P(self.w), K, self.capi.W_MK, P(self.g), P(self.amax),
                                            P(self.amin), P(self.wsel), P(self.xsel), P(self.xg), P(self.wg),
                                            P(self.max_count), P(self.min_count), self.capi.COUNT_HITS, N, K, M,
                                            self.sp)
        assert rc == 0, self.lib.mam_last_error()

    def describe(self):
        """Which kernels the library takes for this layer's forward (asked of the library itself)."""
        buf = ctypes.create_string_buffer(256)
        fn = self.lib.mam_fc_forward_describe
        fn(self._p(self.x), self.K, self._p(self.w), self.K, self.capi.W_MK, self.N, self.K, self.M,
           0 if self.values_only else 1, buf, 256)
        return buf.value.decode()

    def backward_bytes(self):
        N, K, M = self.N, self.K, self.M
        return 4 * (N * K + N * M + 2 * N * M + 2 * N * M + N * K + K * M)


def dense_cpu_baseline(torch, layers_cpu, budget_s, with_backward):
    """Times the pure-PyTorch port on the first `rows` batch rows of every layer."""
    from oracle import torch_port

    def run(rows):
        t0 = time.perf_counter()
        for x, w, g in layers_cpu:
            b = w.T.contiguous()
            _, amax, amin = torch_port.forward(x[:rows], b)
            if with_backward:
                torch_port.backward(x[:rows], b, g[:rows], amax, amin)
        return time.perf_counter() - t0

    n_rows = layers_cpu[0][0].shape[0]
    per_row = run(2) / 2
    rows = int(max(2, min(n_rows, budget_s / max(per_row, 1e-6))))
    dt = run(rows)
    triples = sum(rows * x.shape[1] * w.shape[0] for x, w, _ in layers_cpu)
    return {
        "value": round(triples / dt / 1e9, 4),
        "unit": "GOPS",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": "forward%s of oracle/torch_port.py on the first %d of %d batch rows (%.1f s); rows are "
                  "independent, so GOPS does not depend on the row count"
                  % ("+backward" if with_backward else "", rows, n_rows, dt),
    }


def time_phases(torch, stream, phases, steps, warmup, graph=False):
    """Runs every phase once per step; returns (ms per step by the host clock, ms per phase by events).
    graph: the step is recorded once into a HIP graph and the timed steps are replays of it; the
    per-phase times then come from a second, eager pass."""
    # Clock ramp: the same phases, untimed, whatever --warmup says (a GPU that has been idle runs its first
    # few hundred launches at a lower clock).  Then the counted warm-up.
    global RAMP_REPORT
    calls, t_ramp = 0, time.perf_counter()
    while True:
        for _, fn in phases:
            fn()
        calls += len(phases)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t_ramp
        if (calls >= RAMP_MIN_CALLS and dt >= RAMP_MIN_SECONDS) or dt >= RAMP_MAX_SECONDS:
            break
    RAMP_REPORT = {"ramp_launches": calls, "ramp_ms": round(dt * 1e3, 1)}
    for _ in range(warmup):
        for _, fn in phases:
            fn()
    torch.cuda.synchronize()
    ms_graph = None
    if graph:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _, fn in phases:
                fn()
        for _ in range(min(warmup, 20)):
            g.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            g.replay()
        torch.cuda.synchronize()
        ms_graph = (time.perf_counter() - t0) * 1e3 / steps
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(len(phases) + 1)] for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(steps):
        ev[s][0].record(stream)
        for i, (_, fn) in enumerate(phases):
            fn()
            ev[s][i + 1].record(stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    per_phase = {}
    for i, (label, _) in enumerate(phases):
        ms = sum(e[i].elapsed_time(e[i + 1]) for e in ev) / steps
        per_phase[label] = per_phase.get(label, 0.0) + ms
    return (ms_graph if graph else (t1 - t0) * 1e3 / steps), per_phase


RAMP_REPORT = {}


def valu_roofline(kernel, triples, ms):
    tflops = 3.0 * triples / (ms * 1e-3) / 1e12
    return {"kernel": kernel, "bound": "valu", "achieved": round(tflops, 3), "peak": VALU_PEAK_TFLOPS,
            "unit": "TFLOP/s", "frac": round(tflops / VALU_PEAK_TFLOPS, 4),
            "frac_of_vector_fp32_157.3": round(tflops / VECTOR_FP32_PEAK_TFLOPS, 4), "traffic": None}


def hbm_roofline(kernel, nbytes, ms):
    gbs = nbytes / (ms * 1e-3) / 1e9
    return {"kernel": kernel, "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None, "algorithmic_bytes": nbytes}


def run_dense(torch, capi, lib, dev, args):
    """headline, values_headline, vit_mlp and inference_*: dense layers in (out, in) weight layout."""
    gen = torch.Generator().manual_seed(0)
    wl = args.workload
    if wl in ("headline", "values_headline"):
        N, K, M = 256, 4096, 4096
        x = torch.randn(N, K, generator=gen)
        w = (torch.rand(M, K, generator=gen) * 2 - 1) / 64.0       # U(-1/64, 1/64)
        g = torch.randn(N, M, generator=gen)
        shapes = [(x, w, g)]
        backward, count, values = wl == "headline", wl == "headline", wl == "values_headline"
        text = ("MAM FullyConnected fp32 batch 256 in 4096 out 4096: exact forward with argmax/argmin + "
                "backward (grad_x, grad_W) + selection-count accumulation; x~N(0,1), W~U(-1/64,1/64), "
                "grad_out~N(0,1), seed 0; weight in (out,in) layout") if wl == "headline" else \
               "MAM FullyConnected fp32 batch 256 in 4096 out 4096: values-only forward; x~N(0,1), W~U(-1/64,1/64)"
    elif wl == "config1":
        N, K, M = 64, 784, 256
        x = torch.randn(N, K, generator=gen)
        w = (torch.rand(M, K, generator=gen) * 2 - 1) / 28.0       # Kaiming-uniform(a=sqrt 5), fan_in 784
        g = torch.randn(N, M, generator=gen)
        shapes = [(x, w, g)]
        backward, count, values = True, True, False
        text = ("MAM FullyConnected fp32 batch 64 in 784 out 256 (the small configuration the CPU can run whole): "
                "forward with argmax/argmin + backward + selection count; launch-latency bound")
    elif wl == "vit_mlp":
        N = 12608
        shapes = []
        for K, M in ((768, 3072), (3072, 768)):
            x = torch.randn(N, K, generator=gen)
            w = (torch.rand(M, K, generator=gen) * 2 - 1) / K ** 0.5   # Kaiming-uniform(a=sqrt 5)
            g = torch.randn(N, M, generator=gen)
            shapes.append((x, w, g))
        backward, count, values = True, False, False
        text = ("ViT-B/16-shaped MAM MLP block fp32: 12608 rows, MAM FC 768->3072 then MAM FC 3072->768, each fed "
                "N(0,1) rows; W Kaiming-uniform; forward + backward of both layers")
    else:
        N, K, M = 16384, 4096, int(wl.split("_m")[1])
        x = torch.rand(N, K, generator=gen) * 2 - 1
        w = torch.randn(M, K, generator=gen) * 0.02
        shapes = [(x, w, None)]
        backward, count, values = False, False, False
        text = "MAM inference fp32: batch 16384, in 4096, out %d, forward with argmax/argmin; x~U(-1,1), W~N(0,0.02)" % M

    layers = [Layer(torch, capi, lib, dev, x, w, g, backward, count, values) for x, w, g in shapes]
    phases = []
    for i, L in enumerate(layers):
        phases.append(("forward", L.forward))
    if backward and count and args.fused_count:
        phases.append(("backward_and_selection_count", layers[0].backward_count))
    else:
        if backward:
            for L in reversed(layers):
                phases.append(("backward", L.backward))
        if count:
            phases.append(("selection_count", layers[0].count))
    if wl == "headline":
        # one plain 64 MiB copy kernel: the known-size reference that scales the profiler's
        # FETCH_SIZE / WRITE_SIZE counters when traffic is measured
        calibration_copy = layers[0].max_count.clone()
        del calibration_copy

    stream = torch.cuda.current_stream(dev)
    ms_step, ph = time_phases(torch, stream, phases, args.steps, args.warmup, args.graph)
    triples = sum(L.N * L.K * L.M for L in layers)
    fwd_ms = ph["forward"]
    out = {
        "config": {"workload": text, "name": wl, "layers": [{"N": L.N, "K": L.K, "M": L.M} for L in layers],
                   "launch": "one HIP graph replay per step" if args.graph else "one C-ABI call per phase"},
        "phases_ms": {k: round(v, 5) for k, v in ph.items()},
        "forward_gops": round(triples / (fwd_ms * 1e-3) / 1e9, 2),
    }
    kernel = "; ".join(sorted(set(L.describe() for L in layers))) + " (one forward call per layer)"
    out["roofline"] = valu_roofline(kernel, triples, fwd_ms)
    if wl == "headline":
        out["roofline"]["traffic"] = sum(FORWARD_TRAFFIC_BYTES.values())
        out["roofline"]["traffic_by_kernel"] = FORWARD_TRAFFIC_BYTES
        out["roofline"]["traffic_source"] = "constant from %s, not measured by this run" % TRAFFIC_PROFILE
        # x, w, c, argmax, argmin and the four hand-over planes (w_sel, x_sel)
        out["roofline"]["algorithmic_bytes"] = 4 * (256 * 4096 + 4096 * 4096 + 8 * 256 * 4096)
    fused = "backward_and_selection_count" in ph
    if fused:
        # one call: x_grad, then w_grad and the counters from the same slabs; the index arrays are read by the
        # x_grad kernel and once more by the fused kernel (not a third time by a count kernel)
        L = layers[0]
        both_ms = ph["backward_and_selection_count"]
        nbytes = L.backward_bytes() + 4 * 2 * L.M * L.K
        out["roofline_backward"] = hbm_roofline("mam_bwd_x_kernel + mam_bwd_w_count_kernel (w_grad and hit counts of "
                                                "the same slabs)", nbytes, both_ms)
        out["fwd_bwd_count_gops"] = round(triples / ((fwd_ms + both_ms) * 1e-3) / 1e9, 2)
        backward = count = False
    if backward:
        bwd_ms = ph["backward"]
        out["fwd_bwd_gops"] = round(triples / ((fwd_ms + bwd_ms) * 1e-3) / 1e9, 2)
        out["fwd_bwd_valu_frac"] = round(3.0 * triples / ((fwd_ms + bwd_ms) * 1e-3) / 1e12 / VALU_PEAK_TFLOPS, 4)
        out["roofline_backward"] = hbm_roofline("mam_bwd_x_kernel + mam_bwd_w_vec_kernel",
                                                sum(L.backward_bytes() for L in layers), bwd_ms)
        if wl == "headline":
            out["roofline_backward"]["traffic"] = sum(BACKWARD_TRAFFIC_BYTES.values())
            out["roofline_backward"]["traffic_by_kernel"] = BACKWARD_TRAFFIC_BYTES
            out["roofline_backward"]["traffic_source"] = "constant from %s, not measured by this run" % TRAFFIC_PROFILE
    if count:
        L = layers[0]
        # read both index arrays, read-modify-write both counter arrays once
        out["roofline_selection_count"] = hbm_roofline("selcount_kernel (hits mode)",
                                                       4 * (2 * L.N * L.M + 2 * L.M * L.K), ph["selection_count"])
        out["roofline_selection_count"]["traffic"] = sum(SELCOUNT_TRAFFIC_BYTES.values())
        out["roofline_selection_count"]["traffic_source"] = \
            "constant from %s, not measured by this run" % TRAFFIC_PROFILE
    cpu = None
    if args.cpu_seconds > 0:
        cpu = dense_cpu_baseline(torch, shapes, args.cpu_seconds, backward)
    return triples, ms_step, out, cpu


def run_sparse(torch, capi, lib, dev, args):
    """sparse_d*: CSR forward + backward over a uniformly pruned 4096 x 4096 weight, batch 256."""
    density = {"sparse_d10": 0.10, "sparse_d03": 0.03, "sparse_d01": 0.01}[args.workload]
    N, K, M = 256, 4096, 4096
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(N, K, generator=gen)
    w = torch.randn(M, K, generator=gen) * 0.02
    g = torch.randn(N, M, generator=gen)
    keep = max(1, int(round(density * K)))
    mask = torch.zeros(M, K, dtype=torch.bool)
    for m in range(M):                                   # seeded random subset of columns per row
        mask[m, torch.randperm(K, generator=gen)[:keep]] = True
    dense = w * mask
    csr = dense.to_sparse_csr()
    crow, col, val = (t.to(dev) for t in (csr.crow_indices(), csr.col_indices(), csr.values()))
    nnz = int(val.numel())
    xd, gd = x.to(dev), g.to(dev)
    c = torch.empty((N, M), dtype=torch.float32, device=dev)
    amax = torch.empty((N, M), dtype=torch.int32, device=dev)
    amin = torch.empty((N, M), dtype=torch.int32, device=dev)
    xg = torch.empty((N, K), dtype=torch.float32, device=dev)
    vg = torch.empty((nnz,), dtype=torch.float32, device=dev)
    ws_bytes = lib.mam_csr_fc_forward_workspace(N, K, M)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    wsel = torch.empty((2, N, M), dtype=torch.float32, device=dev)   # selected values, forward -> backward
    psel = torch.empty((2, N, M), dtype=torch.int32, device=dev)     # their positions in col/val
    xsel = torch.empty((2, N, M), dtype=torch.float32, device=dev)   # the selected inputs
    stream = torch.cuda.current_stream(dev)
    sp = ctypes.c_void_p(stream.cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())

    def forward():
        rc = lib.mam_csr_fc_forward(P(xd), K, P(crow), P(col), P(val), None, P(c), P(amax), P(amin), P(wsel),
                                    P(psel), P(xsel), N, K, M, nnz, P(ws), ws_bytes, sp)
        assert rc == 0, lib.mam_last_error()

    def backward():
        rc = lib.mam_csr_fc_backward(P(xd), K, P(crow), P(col), P(val), P(gd), P(amax), P(amin), P(wsel),
                                     P(psel), P(xsel), P(xg), P(vg), N, K, M, nnz, sp)
        assert rc == 0, lib.mam_last_error()

    # one plain 64 MiB copy kernel: the known-size reference that scales the profiler's FETCH_SIZE /
    # WRITE_SIZE counters when traffic is measured
    calibration_src = torch.empty(16 * 1024 * 1024, dtype=torch.float32, device=dev)
    calibration_copy = calibration_src.clone()
    del calibration_src, calibration_copy
    ms_step, ph = time_phases(torch, stream, [("forward", forward), ("backward", backward)], args.steps, args.warmup)
    triples = nnz * N                                    # stored products only
    fwd_bytes = 12 * nnz + 4 * N * K + 12 * N * M + 24 * N * M       # + hand-over arrays
    bwd_bytes = 12 * N * M + 24 * N * M + 4 * N * K + 4 * nnz
    out = {
        "config": {"workload": "Pruned CSR-sparse MAM FullyConnected fp32: 4096x4096 weight, %.0f %% of entries kept "
                               "(seeded random columns per row), W~N(0,0.02), batch 256, x~N(0,1); sparse forward + "
                               "backward; one op = one stored product" % (density * 100),
                   "name": args.workload, "N": N, "K": K, "M": M, "nnz": nnz},
        "phases_ms": {k: round(v, 5) for k, v in ph.items()},
        "forward_gops": round(triples / (ph["forward"] * 1e-3) / 1e9, 2),
        "dense_equivalent_forward_gops": round(N * K * M / (ph["forward"] * 1e-3) / 1e9, 2),
        "roofline": hbm_roofline("transpose_kernel + csr_fwd_kernel", fwd_bytes, ph["forward"]),
        # every stored product fetches its own x value through the vector memory path (64 B per clock and CU):
        # 4 * nnz * N bytes at 256 CUs x 64 B x 2.4 GHz = 39.3 TB/s is the floor of this formulation
        "operand_fetch_bound": {"bytes": 4 * nnz * N, "peak_tbs": 39.3,
                                "floor_ms": round(4 * nnz * N / 39.3e12 * 1e3, 5),
                                "achieved_tbs": round(4.0 * nnz * N / (ph["forward"] * 1e-3) / 1e12, 2)},
        "roofline_backward": hbm_roofline("mam_bwd_x_kernel + csr_bwd_val_kernel", bwd_bytes, ph["backward"]),
    }
    cpu = None
    if args.cpu_seconds > 0:
        # dense-equivalent semantics: the port runs on the densified weight; its GOPS are counted in
        # stored products like `value`
        cpu = dense_cpu_baseline(torch, [(x, dense, g)], args.cpu_seconds, True)
        cpu["value"] = round(cpu["value"] * nnz / (K * M), 4)
        cpu["sample"] += "; densified weight, stored products counted"
    return triples, ms_step, out, cpu


def run_spmm(torch, capi, lib, dev, args):
    """spmm_d*: c = A @ b, A 4096 x 4096 CSR with Bernoulli-kept N(0,1) entries (the reference's own
    generator, test/test_sparse.py:14-17), b dense 4096 x 4096."""
    keep = {"spmm_d30": 0.30, "spmm_d10": 0.10, "spmm_d01": 0.01}[args.workload]
    R = K = C = 4096
    gen = torch.Generator().manual_seed(0)
    a = torch.randn(R, K, generator=gen) * torch.bernoulli(torch.full((R, K), keep), generator=gen)
    b = torch.randn(K, C, generator=gen)
    csr = a.to_sparse_csr()
    crow, col, val = (t.to(dev) for t in (csr.crow_indices(), csr.col_indices(), csr.values()))
    nnz = int(val.numel())
    bd = b.to(dev)
    c = torch.empty((R, C), dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream(dev)
    sp = ctypes.c_void_p(stream.cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())

    def spmm():
        rc = lib.mam_csr_spmm(P(crow), P(col), P(val), P(bd), C, P(c), R, K, C, sp)
        assert rc == 0, lib.mam_last_error()

    # The step is the reference's operator as a user calls it: from one stored entry in eight on it writes
    # the operand out dense and calls the library GEMM, below that it runs the sparse kernel timed beside it.
    csr_dev = torch.sparse_csr_tensor(crow, col, val, size=(R, K))
    op = torch.ops.mamtorch_kernel_sparsev1.cusparsemm
    dense_route = nnz * 8 >= R * K
    ms_step, ph = time_phases(torch, stream, [("spmm", lambda: op(csr_dev, bd))], args.steps, args.warmup)
    _, ph_k = time_phases(torch, stream, [("csr_spmm_kernel", spmm)], max(args.steps // 4, 5), 5)
    _, ph_lib = time_phases(torch, stream, [("torch.sparse.mm", lambda: torch.sparse.mm(csr_dev, bd))],
                            max(args.steps // 10, 5), 5)
    ops = nnz * C
    nbytes = 12 * nnz + 4 * K * C + 4 * R * C
    out = {
        "config": {"workload": "sum-of-products SpMM fp32: A 4096x4096 CSR, %.0f %% of entries stored (Bernoulli mask "
                               "on N(0,1), seed 0), times dense b 4096x4096; one op = one multiply-add"
                               % (keep * 100), "name": args.workload, "R": R, "K": K, "C": C, "nnz": nnz},
        "phases_ms": {k: round(v, 5) for k, v in ph.items()},
        "sparse_kernel_ms": {k: round(v, 5) for k, v in ph_k.items()},
        "library_ms": {k: round(v, 5) for k, v in ph_lib.items()},
        "operand_fetch_tbs": round(4.0 * nnz * C / (ph_k["csr_spmm_kernel"] * 1e-3) / 1e12, 2),
        "roofline": hbm_roofline("csr_to_dense_kernel + library fp32 GEMM" if dense_route else "csr_spmm_kernel",
                                 nbytes, ph["spmm"]),
    }
    cpu = None
    if args.cpu_seconds > 0:
        rows = 256
        t0 = time.perf_counter()
        torch.sparse.mm(a[:rows].to_sparse_csr(), b)
        dt = time.perf_counter() - t0
        cpu = {"value": round(int((a[:rows] != 0).sum()) * C / dt / 1e9, 4), "unit": "GOPS",
               "cores": torch.get_num_threads(), "kind": "port",
               "sample": "torch.sparse.mm on the CPU over the first %d rows of A (%.2f s)" % (rows, dt)}
    return ops, ms_step, out, cpu


def run_spmm_sweep(torch, capi, lib, dev, args):
    """spmm_sweep: the reference's own sparse benchmark grid (test/test_sparse.py:51-101, restated): square
    sizes 128 .. 4096, sparse rates 0.7 .. 0.999, COO and CSR; the operator mamtorch_kernel_sparsev1::cusparsemm
    on fixed operands, with torch.matmul of the dense operand and torch.sparse.mm beside it (events on the
    stream; the reference times with the host clock around fresh random operands)."""
    sizes = [128, 256, 512, 1024, 2048, 4096]
    rates = [0.7, 0.8, 0.9, 0.95, 0.99, 0.999]
    layouts = [("coo", torch.sparse_coo), ("csr", torch.sparse_csr)]
    op = torch.ops.mamtorch_kernel_sparsev1.cusparsemm
    stream = torch.cuda.current_stream(dev)
    steps = min(args.steps, 20)

    def timed(fn, reps):
        for _ in range(3):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record(stream)
        for _ in range(reps):
            fn()
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    # clock ramp on the largest dense product
    big = torch.randn(4096, 4096, device=dev)
    t_ramp = time.perf_counter()
    while time.perf_counter() - t_ramp < RAMP_MIN_SECONDS:
        big @ big
        torch.cuda.synchronize()
    del big
    cells, total_ops, total_ms = [], 0, 0.0
    gen = torch.Generator().manual_seed(0)
    for size in sizes:
        b = torch.randn(size, size, generator=gen).to(dev)
        for rate in rates:
            a = torch.randn(size, size, generator=gen) * torch.bernoulli(torch.full((size, size), 1 - rate), generator=gen)
            ad = a.to(dev)
            nnz = int((a != 0).sum())
            dense_ms = timed(lambda: torch.matmul(ad, b), steps)
            for name, layout in layouts:
                asp = ad.to_sparse(layout=layout)
                ms = timed(lambda: op(asp, b), steps)
                lib_ms = timed(lambda: torch.sparse.mm(asp, b), max(steps // 4, 3))
                dense_route = size >= 64 and nnz * (16 if name == "coo" else 8) >= size * size
                cells.append({"size": size, "sparse_rate": rate, "layout": name, "nnz": nnz,
                              "cusparsemm_ms": round(ms, 5), "torch_matmul_dense_ms": round(dense_ms, 5),
                              "torch_sparse_mm_ms": round(lib_ms, 5),
                              "route": "densify + at::mm" if dense_route else "%s_spmm_kernel" % name})
                total_ops += nnz * size
                total_ms += ms
    biggest = [c for c in cells if c["size"] == 4096 and c["sparse_rate"] == 0.9 and c["layout"] == "csr"][0]
    nb = 12 * biggest["nnz"] + 8 * 4096 * 4096
    out = {
        "config": {"workload": "sum-of-products SpMM sweep of the reference's sparse benchmark: square sizes %s x "
                               "sparse rates %s x {COO, CSR}; A = N(0,1) under a Bernoulli mask, b dense N(0,1); "
                               "one op = one multiply-add of a stored entry; a step = every cell once"
                               % (sizes, rates), "name": args.workload, "launch": "torch.ops calls"},
        "cells": cells,
        "roofline": hbm_roofline("csr_spmm_kernel at 4096, sparse rate 0.9", nb, biggest["cusparsemm_ms"]),
    }
    return total_ops, total_ms, out, None


def run_prune(torch, capi, lib, dev, args):
    """prune_csr: |w| <= threshold goes (90 % of a N(0, 0.02) weight), survivors compacted to CSR."""
    M = K = 4096
    w = (torch.randn(M, K, generator=torch.Generator().manual_seed(0)) * 0.02).to(dev)
    thr = float(torch.sort(w.flatten().abs())[0][int(0.9 * M * K)])
    crow = torch.empty(M + 1, dtype=torch.int64, device=dev)
    stream = torch.cuda.current_stream(dev)
    sp = ctypes.c_void_p(stream.cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    f = ctypes.c_float(thr)

    def offsets():
        rc = lib.mam_prune_row_offsets(P(w), K, capi.PRUNE_MAGNITUDE, None, None, K, f, P(crow), M, K, sp)
        assert rc == 0, lib.mam_last_error()

    offsets()
    nnz = int(crow[M].item())
    col = torch.empty(nnz, dtype=torch.int64, device=dev)
    val = torch.empty(nnz, dtype=torch.float32, device=dev)

    def fill():
        rc = lib.mam_prune_fill_csr(P(w), K, capi.PRUNE_MAGNITUDE, None, None, K, f, P(crow), P(col), P(val), M, K, sp)
        assert rc == 0, lib.mam_last_error()

    # the threshold itself: the element of rank int(0.9 n) of |w| by radix select (3 histogram passes over w),
    # as calls on the stream with the result left on the device; the host reads it once per pruning step
    sel_ws = torch.empty(lib.mam_select_workspace(), dtype=torch.uint8, device=dev)
    sel_out = torch.empty(1, dtype=torch.float32, device=dev)
    rank = (ctypes.c_int64 * 1)(int(0.9 * M * K))

    def threshold():
        rc = lib.mam_select_begin(P(sel_ws), ctypes.c_size_t(sel_ws.numel()), rank, 1, sp)
        for ps in range(3):
            rc = rc or lib.mam_select_accumulate(P(sel_ws), P(w), ctypes.c_int64(K), capi.PRUNE_MAGNITUDE, None, None,
                                                 ctypes.c_int64(K), ctypes.c_int64(M), ctypes.c_int64(K), ps, sp)
            rc = rc or lib.mam_select_advance(P(sel_ws), ps, sp)
        rc = rc or lib.mam_select_result(P(sel_ws), capi.PRUNE_MAGNITUDE, P(sel_out), sp)
        assert rc == 0, lib.mam_last_error()

    threshold()
    assert float(sel_out[0]) == thr, "radix select and sort disagree on the threshold"
    ms_step, ph = time_phases(torch, stream, [("threshold_select", threshold), ("row_offsets", offsets), ("fill", fill)],
                              args.steps, args.warmup)
    # what the reference's statements cost on the same GPU: the sort behind the global rule (torch.quantile refuses
    # 4096 x 4096 elements), the masked assignment, and the library's conversion to CSR
    masked = torch.where(w.abs() > thr, w, torch.zeros_like(w))
    wcopy = w.clone()

    def lib_threshold():
        return torch.sort(w.flatten().abs())[0][int(0.9 * M * K)]

    def lib_mask():
        wcopy[wcopy.abs() <= thr] = 0

    _, ph_lib = time_phases(torch, stream, [("torch.sort threshold", lib_threshold), ("masked assignment", lib_mask),
                                            ("Tensor.to_sparse_csr", lambda: masked.to_sparse_csr())],
                            max(args.steps // 10, 5), 3)
    nbytes = (3 + 2) * 4 * M * K + 8 * (M + 1) + 12 * nnz
    out = {
        "config": {"workload": "magnitude pruning of a 4096x4096 fp32 weight ~N(0,0.02): the threshold (element of rank "
                               "0.9 n of |w|, radix select), then the survivors compacted to CSR (int64 indices); one "
                               "op = one weight examined",
                   "name": args.workload, "M": M, "K": K, "nnz": nnz},
        "phases_ms": {k: round(v, 5) for k, v in ph.items()},
        "library_ms": {k: round(v, 5) for k, v in ph_lib.items()},
        "roofline": hbm_roofline("select hist_kernel x 3 + prune count_kernel + scan_kernel + fill_kernel", nbytes,
                                 ms_step),
    }
    cpu = None
    if args.cpu_seconds > 0:
        wc = w.cpu()
        t0 = time.perf_counter()
        torch.where(wc.abs() > thr, wc, torch.zeros_like(wc)).to_sparse_csr()
        dt = time.perf_counter() - t0
        cpu = {"value": round(M * K / dt / 1e9, 4), "unit": "GOPS", "cores": torch.get_num_threads(), "kind": "port",
               "sample": "mask + Tensor.to_sparse_csr of the whole weight on the CPU (%.2f s)" % dt}
    return M * K, ms_step, out, cpu


def run_reference_script(torch, capi, lib, dev, args):
    """reference_script: what the reference's test script times (test/test.py:186-323), through the operators of
    the reference's names and signatures, b in the (in, out) layout.  Each call is timed between events on the
    stream and, as the script does it, by the host clock around the call and a device synchronize."""
    N, M, K = 128, 4096, 2048
    gen = torch.Generator().manual_seed(0)
    a = torch.randn(N, K, generator=gen).to(dev)
    b = torch.randn(K, M, generator=gen).to(dev)
    c = torch.randn(N, M, generator=gen).to(dev)
    amax = torch.randint(0, K - 1, (N, M), generator=gen, dtype=torch.int32).to(dev)
    amin = torch.randint(0, K - 1, (N, M), generator=gen, dtype=torch.int32).to(dev)
    v1, v4 = torch.ops.mamtorch_kernel_v1, torch.ops.mamtorch_kernel_v4
    phases = [("v1.fullyconnected", lambda: v1.fullyconnected(a, b)),
              ("v4.fullyconnected", lambda: v4.fullyconnected(a, b)),
              ("v4.fullyconnected_fast", lambda: v4.fullyconnected_fast(a, b)),
              ("v4.fullyconnected_backward", lambda: v4.fullyconnected_backward(a, b, c, amax, amin))]
    stream = torch.cuda.current_stream(dev)
    ms_step, ph = time_phases(torch, stream, phases, args.steps, args.warmup)
    _, ph_lib = time_phases(torch, stream, [("torch.matmul", lambda: torch.matmul(a, b))], args.steps, args.warmup)
    wall = {}
    for label, fn in phases + [("torch.matmul", lambda: torch.matmul(a, b))]:
        total = 0.0
        for _ in range(args.steps):
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            total += time.perf_counter() - t0
        wall[label] = round(total * 1e3 / args.steps, 5)
    triples = N * K * M
    out = {
        "config": {"workload": "the reference's own timing loop: a (128, 2048) ~N(0,1) x b (2048, 4096) ~N(0,1), "
                               "(in, out) operand as the reference's operators take it; v1 and v4 forward with "
                               "indices, v4 values-only forward, v4 backward with random indices; one op = one "
                               "multiply-max-min triple of ONE forward (value = triples / time of the four calls)",
                   "name": args.workload, "N": N, "K": K, "M": M, "launch": "torch.ops calls"},
        "phases_ms": {k: round(v, 5) for k, v in ph.items()},
        "host_clock_ms_per_call_with_synchronize": wall,
        "library_ms": {k: round(v, 5) for k, v in ph_lib.items()},
        "roofline": valu_roofline("mamtorch_kernel_v1::fullyconnected (transpose of b + tiling A + merge)", triples,
                                  ph["v1.fullyconnected"]),
    }
    return triples, ms_step, out, None


def run_module(torch, capi, lib, dev, args):
    """module_headline / module_vit_mlp: nn.FullyConnected modules driven the way a training loop drives them
    (mamtorch/nn/v4/fullyconnected.py:133-208 forward, mamtorch/kernel/v4/fullyconnected.py:24-41 autograd):
    forward allocates its outputs, the hand-over planes and the split-K workspace, autograd allocates the
    gradients.  The C-ABI step over the same operands with pre-allocated buffers runs in the same process."""
    import mamtorch

    gen = torch.Generator().manual_seed(0)
    headline = args.workload == "module_headline"
    if headline:
        N = 256
        dims = [(4096, 4096)]
        text = ("mamtorch.nn.FullyConnected(4096, 4096, bias=True, store_args=True, selection_count_mode='hits') "
                "at batch 256: forward + autograd backward (grad_x, grad_W, grad_bias) + "
                "update_selection_count(); x~N(0,1), W~U(-1/64,1/64), grad_out~N(0,1), seed 0")
    else:
        N = 12608
        dims = [(768, 3072), (3072, 768)]
        text = ("ViT-B/16-shaped MAM MLP block through the module: 12608 rows, nn.FullyConnected 768->3072 and "
                "3072->768 (bias=True), each fed N(0,1) rows as in the C-ABI workload; forward + autograd backward")
    layers, shapes = [], []
    for K, M in dims:
        layer = mamtorch.nn.FullyConnected(K, M, bias=True, store_args=headline).to(dev).train()
        if headline:
            layer.selection_count_mode = "hits"
        w = (torch.rand(M, K, generator=gen) * 2 - 1) / K ** 0.5
        x = torch.randn(N, K, generator=gen)
        g = torch.randn(N, M, generator=gen)
        with torch.no_grad():
            layer.weight.copy_(w.to(dev))
        layers.append(layer)
        shapes.append((x, w, g))
    xs = [x.to(dev).requires_grad_(True) for x, _, _ in shapes]
    gs = [g.to(dev) for _, _, g in shapes]
    params = [p for layer in layers for p in layer.parameters()]
    outs = [None] * len(layers)

    def m_forward():
        for p_ in params:
            p_.grad = None
        for x_ in xs:
            x_.grad = None
        for i, layer in enumerate(layers):
            outs[i] = layer(xs[i])

    def m_backward():
        torch.autograd.backward(outs, gs)

    def m_count():
        layers[0].update_selection_count()

    phases = [("forward", m_forward), ("backward", m_backward)]
    if headline:
        layers[0].reset_selection_count()
        phases.append(("selection_count", m_count))
    stream = torch.cuda.current_stream(dev)
    ms_step, ph = time_phases(torch, stream, phases, args.steps, args.warmup)

    # the same operands through the C ABI, buffers allocated once
    cl = [Layer(torch, capi, lib, dev, x, layers[i].weight.detach().cpu(), g, True, headline)
          for i, (x, _, g) in enumerate(shapes)]
    cph = [("forward", L.forward) for L in cl] + [("backward", L.backward) for L in reversed(cl)]
    if headline:
        cph.append(("selection_count", cl[0].count))
    ms_cabi, ph_cabi = time_phases(torch, stream, cph, args.steps, args.warmup)

    triples = sum(N * K * M for K, M in dims)
    bwd_bytes = sum(L.backward_bytes() for L in cl)
    out = {
        "config": {"workload": text, "name": args.workload,
                   "layers": [{"N": N, "K": K, "M": M} for K, M in dims],
                   "launch": "nn.Module forward, torch.autograd.backward, update_selection_count()"},
        "phases_ms": {k: round(v, 5) for k, v in ph.items()},
        "forward_gops": round(triples / (ph["forward"] * 1e-3) / 1e9, 2),
        "c_abi_same_run": {"ms_per_step": round(ms_cabi, 5), "phases_ms": {k: round(v, 5) for k, v in ph_cabi.items()},
                           "value_gops": round(triples / (ms_cabi * 1e-3) / 1e9, 2)},
        "module_overhead": {"ms_per_step": round(ms_step - ms_cabi, 5),
                            "fraction_of_c_abi_step": round((ms_step - ms_cabi) / ms_cabi, 4),
                            "by_phase_ms": {k: round(ph[k] - ph_cabi[k], 5) for k in ph},
                            "what": "per step: at::empty of c, argmax, argmin, the (4,N,M) hand-over tensor and the "
                                    "split-K workspace in the forward; at::empty of both gradients, the bias "
                                    "gradient (mam_bias_grad, one more kernel) and autograd's bookkeeping in the backward"},
        "roofline": valu_roofline("; ".join(sorted(set(L.describe() for L in cl))) + " behind the module",
                                  triples, ph["forward"]),
        "fwd_bwd_gops": round(triples / ((ph["forward"] + ph["backward"]) * 1e-3) / 1e9, 2),
        "fwd_bwd_valu_frac": round(3.0 * triples / ((ph["forward"] + ph["backward"]) * 1e-3) / 1e12 / VALU_PEAK_TFLOPS, 4),
        "roofline_backward": hbm_roofline("mam_bwd_x_kernel + mam_bwd_w_vec_kernel + col_sum_kernel behind autograd",
                                          bwd_bytes, ph["backward"]),
    }
    cpu = None
    if args.cpu_seconds > 0:
        cpu = dense_cpu_baseline(torch, [(x, layers[i].weight.detach().cpu(), g) for i, (x, _, g) in enumerate(shapes)],
                                 args.cpu_seconds, True)
    return triples, ms_step, out, cpu


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed steps after the fixed clock ramp (at least %d phase calls, always run)" % RAMP_MIN_CALLS)
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU baseline budget; 0 skips it")
    ap.add_argument("--workload", choices=WORKLOADS, default="headline")
    ap.add_argument("--fused-count", action="store_true",
                    help="headline / config1: backward and selection count as ONE call (mam_fc_backward_count)")
    ap.add_argument("--graph", action="store_true",
                    help="dense workloads: record one step into a HIP graph and time replays of it")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the MAM hot path has no multi-GPU part in this build "
              "(--gpus %d refused)" % args.gpus, file=sys.stderr)
        sys.exit(2)
    small = args.workload in ("headline", "config1", "values_headline", "prune_csr", "reference_script",
                              "module_headline") \
        or args.workload.startswith("sparse")
    if args.workload.startswith("spmm"):
        args.steps = 50 if args.steps is None else args.steps
        args.warmup = 20 if args.warmup is None else args.warmup
    if args.steps is None:
        args.steps = 500 if small else 20
    if args.warmup is None:
        args.warmup = 20 if small else 5

    import torch

    import __graft_entry__

    __graft_entry__.ensure_built()      # builds only when nothing is built yet
    from mamtorch_amd import capi

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the MAM operators have no CPU path)", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    lib = capi.lib()
    run = run_sparse if args.workload.startswith("sparse") else run_spmm_sweep if args.workload == "spmm_sweep" \
        else run_spmm if args.workload.startswith("spmm") \
        else run_prune if args.workload == "prune_csr" \
        else run_reference_script if args.workload == "reference_script" \
        else run_module if args.workload.startswith("module_") else run_dense
    triples, ms_step, extra, cpu = run(torch, capi, lib, dev, args)

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
    }
    out.update(extra)
    out.update(RAMP_REPORT)
    props = torch.cuda.get_device_properties(dev)
    cu_c, khz_c = ctypes.c_int(0), ctypes.c_int(0)
    lib.mam_device_info(ctypes.byref(cu_c), ctypes.byref(khz_c))      # what the device itself reports
    cus = int(cu_c.value) or int(props.multi_processor_count)
    mhz = khz_c.value / 1e3
    out["device"] = {"name": props.name, "compute_units": cus, "max_clock_mhz": mhz,
                     "valu_peak_from_device_tflops": round(cus * 128 * mhz * 1e6 / 1e12, 2) if mhz else None,
                     "peaks_used": {"valu_fp32_no_fma_tflops": VALU_PEAK_TFLOPS,
                                    "vector_fp32_tflops": VECTOR_FP32_PEAK_TFLOPS, "hbm_gbs": HBM_PEAK_GBS}}
    out["cpu_baseline"] = cpu
    print(json.dumps(out))


if __name__ == "__main__":
    main()
