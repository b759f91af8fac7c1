#!/usr/bin/env python3
"""Benchmark of the W4A4H MUL_MAT hot path on one MI355X.

A step is one whole operator call (online Hadamard + activation quantizer + product + fp32 epilogue) on a
synthetic problem whose inputs are resident in HBM. The headline workload is the decode shape the target is
stated on: W4A4H, K = 5120, N = 17408, M = 1, reported as GB/s of algorithmic bytes
(N*K/2 codes + 4N scales + 4MK activations in + 4MN out). Successive steps rotate through enough distinct copies
of the weight to exceed the 256 MB Infinity Cache, so the codes come from HBM.

Prints one JSON line. Besides the contract fields it carries
  roofline     : the product kernel alone (HIP events around back-to-back launches on the launch stream),
  cpu_baseline : the CPU oracle (a bit-identical restatement of the ggml-cpu reference path) on the host cores,
  extra        : the same measurements for the other benchmark shapes (M = 2048 prefill as TOPS against the dense
                 int8 MFMA peak, the N = 5120 decode shapes, the K = 17408 down projection) and the seven matmuls of
                 one transformer layer at 16 tokens and at one token, run in the layer's dataflow.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
# HBM bytes per launch of the headline product kernel: rocprofv3 FETCH_SIZE 21,923.0 KiB / 0.500 (scale from a plain
# copy of known size) + WRITE_SIZE 748.0 KiB / 1.000, from the runs summarized in profiles/gemv_m1_k5120_n17408.md
HEADLINE_TRAFFIC_BYTES = int((21923.0 / 0.500 + 748.0) * 1024)
INT8_PEAK_TOPS = 5000.0      # MI355X dense int8 MFMA


def algorithmic_bytes(K, N, M):
    return N * K // 2 + 4 * N + 4 * M * K + 4 * M * N


class Problem:
    """One (K, N, M) W4A4H problem with rotating weight copies and a preallocated workspace."""

    def __init__(self, K, N, M, act_kind, clip, seed, min_rotate_bytes=320 << 20, dev="cuda:0"):
        import numpy as np
        import torch
        import ruquant_amd as rq
        from ruquant_amd import synth
        self.K, self.N, self.M = K, N, M
        self.rq, self.torch = rq, torch
        self.type = rq.TYPE_W4A4H
        self.blocks = synth.random_weight_blocks(N, K, seed, self.type, clip=clip if clip != 1.0 else 0.0)
        self.x_host = synth.activations(act_kind, M, K, seed)
        self.weight = rq.W4A4Weight(self.blocks, self.type, dev, keep_blocks=False)
        self.clip = float(np.float32(clip))
        n_copies = max(1, -(-min_rotate_bytes // (N * K // 2)))
        self.prepared = [self.weight.prepared] + [self.weight.prepared.clone() for _ in range(n_copies - 1)]
        self.x = torch.from_numpy(self.x_host).to(dev)
        self.y = torch.empty((M, N), dtype=torch.float32, device=dev)
        self.ws = self.weight.workspace(M)
        self.L = rq.load_library()
        self.i = 0
        self.graphs = {}
        torch.cuda.synchronize()

    def call(self, stages=3):
        import ctypes
        p = self.prepared[self.i % len(self.prepared)]
        self.i += 1
        rc = self.L.rq_w4a4_mul_mat_stages(self.type, p.data_ptr(), self.K, self.N, self.x.data_ptr(), self.K, self.M,
                                           self.y.data_ptr(), self.N, self.clip, self.K, self.ws.data_ptr(),
                                           self.ws.numel(), ctypes.c_void_p(self.torch.cuda.current_stream().cuda_stream),
                                           stages)
        if rc != 0:
            raise RuntimeError("rq_w4a4_mul_mat_stages failed: %d" % rc)

    def timed(self, steps, warmup, stages=3):
        """ms per call over exactly `steps` back-to-back calls after `warmup` untimed ones. The calls are captured
        into one HIP graph (the operator is graph-safe by contract) so the host's per-call cost does not pace the GPU;
        the eager wall time per call is returned beside it."""
        torch = self.torch
        if stages == 2:
            self.call(1)             # fill the workspace once; the product stage leaves its scratch clean
        for _ in range(max(warmup, 1)):
            self.call(stages)
        torch.cuda.synchronize()
        key = (steps, stages)
        if key not in self.graphs:
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                for _ in range(steps):
                    self.call(stages)
            self.graphs[key] = g
            g.replay()               # first replay uploads the graph
            torch.cuda.synchronize()
        g = self.graphs[key]
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        g.replay()
        e1.record()
        torch.cuda.synchronize()
        gpu_ms = e0.elapsed_time(e1) / steps
        t0 = time.perf_counter()
        for _ in range(steps):
            self.call(stages)
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
        return gpu_ms, wall_ms

    def median_timed(self, steps, warmup, stages, batches=7):
        vals = sorted(self.timed(steps, warmup if b == 0 else 2, stages)[0] for b in range(batches))
        return vals[len(vals) // 2]

    def check(self, oracle):
        import numpy as np
        self.call(3)
        self.torch.cuda.synchronize()
        want = oracle.mul_mat(self.type, self.blocks, self.x_host, self.clip, n_rot=self.K)
        got = self.y.cpu().numpy()
        return bool((got.view(np.uint32) == want.view(np.uint32)).all())


class Layer:
    """The seven W4A4H matmuls of one transformer layer at M tokens, in the layer's dataflow: q, k, v <- x0 (one
    fused call: the three weights share one rotation + quantization of x0); o <- q's output; gate, up <- o's output
    (fused); down <- up's output. Clip 1.0, whole-row rotations (H20xH256, H12xH512 for o, H68xH256 for down). Two
    sets of weights alternate so that successive layers read 341 MB of codes, more than the Infinity Cache holds."""

    SHAPES = [("q", 5120, 6144), ("k", 5120, 1024), ("v", 5120, 1024), ("o", 6144, 5120), ("gate", 5120, 17408),
              ("up", 5120, 17408), ("down", 17408, 5120)]

    def __init__(self, M, seed=1, copies=2, dev="cuda:0"):
        import torch
        import ruquant_amd as rq
        from ruquant_amd import synth
        self.rq, self.torch, self.M = rq, torch, M
        self.sets = []
        for c in range(copies):
            ws = {}
            for i, (name, K, N) in enumerate(self.SHAPES):
                blocks = synth.random_weight_blocks(N, K, seed + i, rq.TYPE_W4A4H, clip=0.0)
                ws[name] = rq.W4A4Weight(blocks, rq.TYPE_W4A4H, dev, keep_blocks=False)
            self.sets.append(ws)
        self.x0 = torch.from_numpy(synth.activations("normal", M, 5120, seed)).to(dev)
        self.out = {name: torch.empty((M, N), dtype=torch.float32, device=dev) for name, K, N in self.SHAPES}
        L = rq.load_library()
        w = self.sets[0]
        self.ws = torch.empty(max([L.rq_w4a4_workspace_bytes(rq.TYPE_W4A4H, K, N, M) for _, K, N in self.SHAPES] +
                                  [rq.fused_workspace_bytes([w["q"], w["k"], w["v"]], M),
                                   rq.fused_workspace_bytes([w["gate"], w["up"]], M)]),
                              dtype=torch.uint8, device=dev)
        self.code_bytes = sum(K * N // 2 for _, K, N in self.SHAPES)
        self.bytes = sum(algorithmic_bytes(K, N, M) for _, K, N in self.SHAPES)
        self.ops = sum(2 * M * K * N for _, K, N in self.SHAPES)
        self.i = 0

    def call(self, fused=True):
        w = self.sets[self.i % len(self.sets)]
        self.i += 1
        rq, o = self.rq, self.out
        if fused:
            rq.mul_mat_fused([w["q"], w["k"], w["v"]], self.x0, outs=[o["q"], o["k"], o["v"]], workspace=self.ws)
        else:
            for n in ("q", "k", "v"):
                rq.mul_mat(w[n], self.x0, out=o[n], workspace=self.ws)
        rq.mul_mat(w["o"], o["q"], out=o["o"], workspace=self.ws)
        if fused:
            rq.mul_mat_fused([w["gate"], w["up"]], o["o"], outs=[o["gate"], o["up"]], workspace=self.ws)
        else:
            for n in ("gate", "up"):
                rq.mul_mat(w[n], o["o"], out=o[n], workspace=self.ws)
        rq.mul_mat(w["down"], o["up"], out=o["down"], workspace=self.ws)

    def timed(self, steps, warmup, fused=True):
        torch = self.torch
        for _ in range(max(warmup, 1)):
            self.call(fused)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(steps):
                self.call(fused)
        g.replay()
        torch.cuda.synchronize()
        vals = []
        for _ in range(5):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            g.replay()
            e1.record()
            torch.cuda.synchronize()
            vals.append(e0.elapsed_time(e1) / steps)
        return sorted(vals)[len(vals) // 2]

    def measure(self, steps, warmup):
        fused_ms = self.timed(steps, warmup, True)
        plain_ms = self.timed(steps, warmup, False)
        return {"M": self.M, "matmuls": 7, "code_bytes": self.code_bytes, "layer_us": round(fused_ms * 1e3, 2),
                "layer_gbs": round(self.bytes / fused_ms / 1e6, 1),
                "layer_frac_of_hbm_peak": round(self.bytes / fused_ms / 1e6 / HBM_PEAK_GBS, 4),
                "layer_tops": round(self.ops / fused_ms / 1e9, 2),
                "layer_us_seven_separate_calls": round(plain_ms * 1e3, 2)}


def cpu_baseline(oracle, prob, budget_s=12.0, max_reps=1500):   # about 20 core-seconds on 16 threads
    threads = min(os.cpu_count() or 1, 16)
    reps, t0 = 0, time.perf_counter()
    while True:
        oracle.mul_mat(prob.type, prob.blocks, prob.x_host, prob.clip, n_rot=prob.K, n_threads=threads)
        reps += 1
        el = time.perf_counter() - t0
        if el > budget_s or reps >= max_reps:
            break
    return el / reps, reps, threads


def measure(prob, steps, warmup, bound):
    op_ms, wall_ms = prob.timed(steps, warmup, 3)
    kern_ms = prob.median_timed(steps, warmup, 2)
    act_ms = prob.median_timed(steps, warmup, 1)
    K, N, M = prob.K, prob.N, prob.M
    out = {"K": K, "N": N, "M": M, "op_us": round(op_ms * 1e3, 3), "op_eager_wall_us": round(wall_ms * 1e3, 3),
           "product_kernel_us": round(kern_ms * 1e3, 3), "activation_kernel_us": round(act_ms * 1e3, 3)}
    if bound == "hbm":
        b = algorithmic_bytes(K, N, M)
        out.update(op_gbs=round(b / op_ms / 1e6, 1), kernel_gbs=round(b / kern_ms / 1e6, 1),
                   kernel_frac_of_hbm_peak=round(b / kern_ms / 1e6 / HBM_PEAK_GBS, 4),
                   op_frac_of_hbm_peak=round(b / op_ms / 1e6 / HBM_PEAK_GBS, 4))
    else:
        ops = 2.0 * M * N * K
        out.update(op_tops=round(ops / op_ms / 1e9, 1), kernel_tops=round(ops / kern_ms / 1e9, 1),
                   kernel_frac_of_int8_peak=round(ops / kern_ms / 1e9 / INT8_PEAK_TOPS, 4),
                   op_frac_of_int8_peak=round(ops / op_ms / 1e9 / INT8_PEAK_TOPS, 4))
    return out, op_ms, kern_ms


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-extra", action="store_true", help="only the headline workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy 10 times (scale for FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--shapes", default="", help="comma-separated names of the extra shapes to run (default: all)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this operator is measured on one GPU; --gpus %d is not a configuration of this build "
              "(the op shards along N with no exchange between GPUs)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    import ruquant_amd as rq
    rq.load_library()   # fails loudly when the HIP library has not been built

    if args.copy_calibration:
        src = torch.ones(64 << 20, dtype=torch.float32, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(10):
            torch.mul(src, 1.0, out=dst)     # a plain elementwise copy kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    K, N, M = 5120, 17408, 1
    head = Problem(K, N, M, "outlier_channels", 0.9, seed=2)
    res, op_ms, kern_ms = measure(head, args.steps, args.warmup, "hbm")
    b = algorithmic_bytes(K, N, M)

    cpu = None
    parity = None
    if not args.no_cpu:
        from oracle import rq_oracle
        parity = head.check(rq_oracle)
        sec, reps, threads = cpu_baseline(rq_oracle, head)
        cpu = {"value": round(b / sec / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
               "sample": "%d whole-op passes of the same K=%d N=%d M=%d problem (%.2f ms each), CPU oracle, "
                         "two-phase threading" % (reps, K, N, M, sec * 1e3)}

    extra = {"headline": res}
    if not args.no_extra:
        shapes = [
            ("decode_k5120_n5120_m1", 5120, 5120, 1, "outlier_channels", 0.9, "hbm"),
            ("decode_k5120_n5120_m8", 5120, 5120, 8, "outlier_channels", 0.9, "hbm"),
            ("down_k17408_n5120_m1", 17408, 5120, 1, "relu2", 1.0, "hbm"),
            ("down_k17408_n5120_m16", 17408, 5120, 16, "relu2", 1.0, "hbm"),
            ("prefill_k5120_n17408_m64", 5120, 17408, 64, "student_t4", 0.85, "hbm"),
            ("prefill_k5120_n17408_m512", 5120, 17408, 512, "student_t4", 0.85, "mfma"),
            ("prefill_k5120_n17408_m2048", 5120, 17408, 2048, "student_t4", 0.85, "mfma"),
            ("down_k17408_n5120_m2048", 17408, 5120, 2048, "relu2", 1.0, "mfma"),
        ]
        want = [w for w in args.shapes.split(",") if w]
        for name, k, n, m, kind, clip, bound in shapes:
            if want and name not in want:
                continue
            head = None
            torch.cuda.empty_cache()
            head = None
            head = Problem(k, n, m, kind, clip, seed=3)
            steps = args.steps if m <= 64 else max(5, args.steps // 10)
            extra[name], _, _ = measure(head, steps, min(args.warmup, steps), bound)

        for name, m in (("layer_m16", 16), ("layer_m1", 1)):
            if not want or name in want:
                head = None
                torch.cuda.empty_cache()
                layer = Layer(m)
                extra[name] = layer.measure(max(5, args.steps // 4), 3)
                del layer

    line = {
        "metric": "w4a4h_matmul_gbps_m1", "value": round(b / op_ms / 1e6, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(op_ms, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "i4xi4->i32",
        "data": "synthetic",
        "config": {"workload": "W4A4H MUL_MAT K=5120 N=17408 M=1 (Hadamard H20xH256, clip 0.9 from pad[1], "
                               "outlier-channel activations), whole op, weights rotated over >256 MB",
                   "algorithmic_bytes": b},
        "roofline": {"bound": "hbm", "achieved": round(b / kern_ms / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(b / kern_ms / 1e6 / HBM_PEAK_GBS, 4), "traffic": HEADLINE_TRAFFIC_BYTES,
                     "kernel": "rq_gemv_kernel<1, 4, 1>", "kernel_us": round(kern_ms * 1e3, 3)},
        "cpu_baseline": cpu,
        "parity_vs_oracle": parity,
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
