#!/usr/bin/env python3
"""Benchmark of the W4A4H MUL_MAT hot path on one MI355X.

A step is one whole operator call (online Hadamard + activation quantizer + product + fp32 epilogue) on a
synthetic problem whose inputs are resident in HBM. The headline workload is the decode shape the target is
stated on: W4A4H, K = 5120, N = 17408, M = 1, reported as GB/s of algorithmic bytes
(N*K/2 codes + 4N scales + 4MK activations in + 4MN out). Successive steps rotate through enough distinct copies
of the weight to exceed the 256 MB Infinity Cache, so the codes come from HBM.

Prints one JSON line. Besides the contract fields it carries
  roofline       : the product kernel of the headline alone (HIP events around back-to-back launches on the launch
                   stream), against the HBM peak,
  roofline_m2048 : the tiled MFMA GEMM alone at M = 2048 (K = 5120, N = 17408), against the dense int8 MFMA peak: the
                   second half of the metric,
  cpu_baseline   : the CPU oracle (a bit-identical restatement of the ggml-cpu reference path) on the host cores, on
                   the headline problem,
  cpu_baseline_m2048 : one whole pass of the same oracle over the M = 2048 problem (its result is also what the GPU's
                   output of that problem is compared with, bit for bit),
  extra          : the same measurements for the other benchmark shapes (the N = 5120 decode shapes, the K = 17408 down
                   projection, the reference's perf-mode shape 6144 x 5120), the seven matmuls of one transformer
                   layer at 16 tokens and at one token, run in the layer's dataflow, and `peaks`: what this machine
                   delivers to plain probe kernels in the same run (a streaming read of the headline's byte count, a
                   pure MFMA loop of every form the kernels use or were weighed against, vector-ALU instructions
                   beside MFMAs in one wavefront and in two wavefronts that share a SIMD, an empty launch).
Every time is the median over 11 batches of back-to-back launches captured in one HIP graph.
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
INT8_PEAK_TOPS = 5000.0      # MI355X dense int8 MFMA
# HBM bytes per launch of the headline's dominant kernel come from the committed rocprofv3 counter summary (FETCH_SIZE
# and WRITE_SIZE passes, each scaled by a plain copy of known size): the line "traffic_bytes_per_launch: <n>" in it
HEADLINE_PROFILE = os.path.join(ROOT, "profiles", "decode_m1_k5120_n17408.md")


GEMM_PROFILE = os.path.join(ROOT, "profiles", "rq_gemm6_kernel_m2048_m512.md")   # "traffic_bytes_per_launch_m2048: <n>"


def profiled_traffic_bytes(path=HEADLINE_PROFILE, key="traffic_bytes_per_launch:"):
    try:
        with open(path) as f:
            for line in f:
                if line.startswith(key):
                    return int(line.split(":")[1].split()[0])
    except OSError:
        pass
    return None


def algorithmic_bytes(K, N, M):
    return N * K // 2 + 4 * N + 4 * M * K + 4 * M * N


class Problem:
    """One (K, N, M) W4A4H problem with rotating weight copies and a preallocated workspace."""

    def __init__(self, K, N, M, act_kind, clip, seed, min_rotate_bytes=320 << 20, dev="cuda:0", type_=None):
        import numpy as np
        import torch
        import ruquant_amd as rq
        from ruquant_amd import synth
        self.K, self.N, self.M = K, N, M
        self.rq, self.torch = rq, torch
        self.type = rq.TYPE_W4A4H if type_ is None else type_
        self.blocks = synth.random_weight_blocks(N, K, seed, self.type, clip=clip if clip != 1.0 else 0.0)
        self.x_host = synth.activations(act_kind, M, K, seed)
        self.weight = rq.W4A4Weight(self.blocks, self.type, dev, keep_blocks=False)
        self.clip = float(np.float32(clip))
        # bytes of a prepared weight that one call reads: the int4 codes, or the fp6 plane of the wide-batch kernel
        fp6 = M > 64 and os.environ.get("RQ_GEMM_FP6", "1") != "0"
        n_copies = max(1, -(-min_rotate_bytes // (N * K * 3 // 4 if fp6 else N * K // 2)))
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
        # Untimed passes of the same graph go out right in front of the timed one, with no host wait between them,
        # until about 3 ms of work precede it: the eager warm-up calls above are paced by the host, and a burst of a
        # fraction of a millisecond after such a stretch runs below the clocks that a busy device settles at (20
        # one-token calls: 11.0 us each cold, 10.6 us behind 3 ms of the same work; 200 calls in one pass: 10.3). The timed
        # interval is exactly `steps` calls, between two events on the stream, with host synchronization before the
        # first pass and after the timed one.
        t0 = time.perf_counter()
        g.replay()
        torch.cuda.synchronize()
        one_pass = max(time.perf_counter() - t0, 1e-5)
        for _ in range(min(int(3e-3 / one_pass), 200)):
            g.replay()
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

    def stage_mask(self):
        """which stages launch kernels for this problem (a one-token call of the single-launch kernel: stage 2 only)"""
        return self.L.rq_w4a4_stage_mask(self.type, self.K, self.M, self.K)

    def median_timed(self, steps, warmup, stages, batches=11):
        vals = sorted(self.timed(steps, warmup if b == 0 else 2, stages)[0] for b in range(batches))
        return vals[len(vals) // 2]

    def check(self, oracle, want=None):
        import numpy as np
        self.call(3)
        self.torch.cuda.synchronize()
        if want is None:
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
        self.shared = rq.SharedActivation(self.ws)
        self.code_bytes = sum(K * N // 2 for _, K, N in self.SHAPES)
        self.bytes = sum(algorithmic_bytes(K, N, M) for _, K, N in self.SHAPES)
        self.ops = sum(2 * M * K * N for _, K, N in self.SHAPES)
        self.i = 0

    def call(self, fused=True):
        w = self.sets[self.i % len(self.sets)]
        self.i += 1
        rq, o = self.rq, self.out
        if fused == "shared":
            # seven separate calls, but q / k / v and gate / up share one rotation + quantization of their x (the
            # reference's activation cache)
            sa = self.shared
            sa.begin()
            for n, src in (("q", self.x0), ("k", self.x0), ("v", self.x0), ("o", o["q"]), ("gate", o["o"]),
                           ("up", o["o"]), ("down", o["up"])):
                sa.mul_mat(w[n], src, o[n])
            return
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
            g.replay()   # untimed, right in front of the timed pass (as in Problem.timed)
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
        shared_ms = self.timed(steps, warmup, "shared")
        return {"M": self.M, "matmuls": 7, "code_bytes": self.code_bytes, "layer_us": round(fused_ms * 1e3, 2),
                "layer_gbs": round(self.bytes / fused_ms / 1e6, 1),
                "layer_frac_of_hbm_peak": round(self.bytes / fused_ms / 1e6 / HBM_PEAK_GBS, 4),
                "layer_tops": round(self.ops / fused_ms / 1e9, 2),
                "layer_us_seven_separate_calls": round(plain_ms * 1e3, 2),
                "layer_us_seven_calls_shared_activation": round(shared_ms * 1e3, 2)}


def host_cores():
    """(logical CPUs the machine reports, CPUs this process may run on)."""
    n = os.cpu_count() or 1
    try:
        usable = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        usable = n
    return n, usable


def cpu_baseline(oracle, prob, budget_s=12.0, max_reps=1500):   # about 20 core-seconds on 16 threads
    threads = min(host_cores()[1], 16)
    reps, t0 = 0, time.perf_counter()
    while True:
        oracle.mul_mat(prob.type, prob.blocks, prob.x_host, prob.clip, n_rot=prob.K, n_threads=threads)
        reps += 1
        el = time.perf_counter() - t0
        if el > budget_s or reps >= max_reps:
            break
    return el / reps, reps, threads


def cpu_one_pass(oracle, prob):
    """one whole pass of the oracle over `prob` on the host's cores: (seconds, threads, result)"""
    threads = min(host_cores()[1], 16)
    t0 = time.perf_counter()
    want = oracle.mul_mat(prob.type, prob.blocks, prob.x_host, prob.clip, n_rot=prob.K, n_threads=threads)
    return time.perf_counter() - t0, threads, want


def measure(prob, steps, warmup, bound):
    _, wall_ms = prob.timed(steps, warmup, 3)
    op_ms = prob.median_timed(steps, 2, 3)
    kern_ms = prob.median_timed(steps, warmup, 2)
    # the activation side has launches of its own unless the single-launch kernel takes the call (then: null)
    act_ms = prob.median_timed(steps, warmup, 1) if prob.stage_mask() & 1 else None
    K, N, M = prob.K, prob.N, prob.M
    out = {"K": K, "N": N, "M": M, "op_us": round(op_ms * 1e3, 3), "op_eager_wall_us": round(wall_ms * 1e3, 3),
           "product_kernel_us": round(kern_ms * 1e3, 3),
           "activation_kernel_us": None if act_ms is None else round(act_ms * 1e3, 3)}
    if prob.type != prob.rq.TYPE_W4A4H:
        out["type"] = "W4A4"
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


def machine_peaks(torch, rq, code_bytes, batches=5):
    """What plain probe kernels reach on this machine, measured like the operator (graph-captured batches between
    events): see rq_probe in include/rq_probe.h (librq_probe.so, a library of its own)."""
    import ctypes
    L = rq.load_probe_library()
    dev = "cuda:0"
    cus = torch.cuda.get_device_properties(0).multi_processor_count

    def timed(fn, n):
        for i in range(2):
            fn(i)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(n):
                fn(i)
        g.replay()
        torch.cuda.synchronize()
        vals = []
        for _ in range(batches):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            g.replay()
            e1.record()
            torch.cuda.synchronize()
            vals.append(e0.elapsed_time(e1) / n * 1e3)
        return sorted(vals)[len(vals) // 2]

    def probe(buf, kind, a0, a1=0, a2=0, a3=0, off=0, nbytes=None):
        rc = L.rq_probe(kind, a0, a1, a2, a3, buf.data_ptr() + off, buf.numel() - off if nbytes is None else nbytes,
                        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        if rc != 0:
            raise RuntimeError("rq_probe(%d) failed: %d" % (kind, rc))

    out = {"compute_units": cus}
    small = torch.zeros(1 << 16, dtype=torch.uint8, device=dev)
    out["empty_launch_us"] = round(timed(lambda i: probe(small, 0, 1088), 50), 3)

    # streaming read of the headline's code bytes, rotating over more than the memory-side cache holds
    copies = max(2, -(-(320 << 20) // code_bytes))
    big = torch.ones(copies * code_bytes // 4, dtype=torch.int32, device=dev).view(torch.uint8)
    best = None
    for loads in (5, 10):
        if code_bytes % (loads * 4096):
            continue
        us = timed(lambda i: probe(big, 1, code_bytes, loads, 0, off=(i % copies) * code_bytes, nbytes=code_bytes), 3 * copies)
        if best is None or us < best[0]:
            best = (us, loads)
    if best:
        out["stream_read"] = {"bytes": code_bytes, "us": round(best[0], 3), "gbs": round(code_bytes / best[0] / 1e3, 1),
                              "loads_in_flight_per_thread": best[1], "source": "HBM (%d rotating buffers)" % copies}
        us = timed(lambda i: probe(big, 1, code_bytes, best[1], 0, off=0, nbytes=code_bytes), 24)
        out["stream_read_cache_resident"] = {"bytes": code_bytes, "us": round(us, 3), "gbs": round(code_bytes / us / 1e3, 1)}
        nb = copies * code_bytes // (best[1] * 4096) * (best[1] * 4096)
        us = timed(lambda i: probe(big, 1, nb, best[1], 0, off=0, nbytes=nb), 4)
        out["stream_read_large"] = {"bytes": nb, "us": round(us, 3), "gbs": round(nb / us / 1e3, 1)}
    del big

    # matrix pipe and vector ALU: workgroups of 8 wavefronts (two per SIMD), one workgroup per compute unit
    ops_per_mfma = 16 * 16 * 64 * 2
    mi, vi = 2000, 1000

    def mix(sub, valu_op=0, one_wave_per_simd=False, m=mi, v=vi, form=0):
        return timed(lambda i: probe(small, 2, sub | valu_op << 8 | (1 << 16 if one_wave_per_simd else 0) | form << 20,
                                     cus, m, v), 4)

    simds = cus * 4
    t = mix(3)
    out["mfma_i8_16x16x64_tops_one_wavefront_per_simd"] = round(cus * 4 * mi * 16 * ops_per_mfma / t / 1e6, 1)
    out["mfma_ns_per_instruction_per_simd"] = round(t * 1e3 / (mi * 16), 3)
    t = mix(0)
    out["mfma_i8_16x16x64_tops_two_wavefronts_per_simd"] = round(cus * 8 * mi * 16 * ops_per_mfma / t / 1e6, 1)
    for op, name in ((0, "v_add_u32"), (1, "v_ashrrev_i32"), (2, "v_mul_i32_i24"), (3, "v_dot8c_i32_i4"),
                     (4, "v_fma_f32"), (5, "v_add_f32")):
        t1, t2 = mix(4, op), mix(1, op)
        out["valu_ns_per_instruction_per_simd_%s" % name] = {"one_wavefront": round(t1 * 1e3 / (vi * 128), 3),
                                                             "two_wavefronts": round(t2 * 1e3 / (2 * vi * 128), 3)}
    # one wavefront per SIMD issues only MFMAs, a second one on the same SIMD only v_add_u32
    t_m, t_v, t_both = mix(3), mix(4), mix(2)
    out["mfma_wavefront_beside_valu_wavefront_us"] = {"mfma_alone": round(t_m, 1), "valu_alone": round(t_v, 1),
                                                      "together": round(t_both, 1), "sum": round(t_m + t_v, 1)}
    # two wavefronts per SIMD of each kind (two workgroups per compute unit): the vector ALU at its full issue rate
    def mix2(sub):
        return timed(lambda i: probe(small, 2, sub, 2 * cus, mi, vi), 4)
    t_m, t_v, t_both = mix2(3), mix2(4), mix2(2)
    out["two_mfma_wavefronts_beside_two_valu_wavefronts_us"] = {"mfma_alone": round(t_m, 1), "valu_alone": round(t_v, 1),
                                                                "together": round(t_both, 1), "sum": round(t_m + t_v, 1)}
    # one wavefront interleaving 1 MFMA with 8 independent v_add_u32 (two such wavefronts per SIMD)
    t = mix(5, 0, False, mi // 4, 0)
    out["same_wavefront_1_mfma_8_valu_ns_per_mfma_per_simd"] = round(t * 1e3 / (2 * (mi // 4) * 16), 3)
    out["same_wavefront_1_mfma_8_valu_tops"] = round(cus * 8 * (mi // 4) * 16 * ops_per_mfma / t / 1e6, 1)
    # The other MFMA forms: alone (two wavefronts per SIMD), one MFMA wavefront beside one v_fma_f32 wavefront on every
    # SIMD, and one wavefront interleaving each MFMA with 16 v_fma_f32 (what the fp6 GEMM's fold does per 32 x 32 tile
    # and group). Ops per instruction: 32 x 32 x 32 x 2 (int8), 32 x 32 x 64 x 2 (f8f6f4).
    forms = {}
    m2 = mi // 4
    for form, name, ops in ((1, "v_mfma_i32_32x32x32_i8", 65536), (2, "v_mfma_f32_32x32x64_f8f6f4_fp8", 131072),
                            (3, "v_mfma_f32_32x32x64_f8f6f4_fp6", 131072)):
        t_alone = mix(0, 4, False, m2, vi, form)
        t_m, t_v, t_both = mix(3, 4, False, m2, vi, form), mix(4, 4, False, m2, vi, form), mix(2, 4, False, m2, vi, form)
        t_16 = mix(6, 4, False, m2 // 2, 0, form)
        forms[name] = {
            "ns_per_instruction_per_simd": round(t_alone * 1e3 / (2 * m2 * 16), 3),
            "tops": round(cus * 8 * m2 * 16 * ops / t_alone / 1e6, 1),
            "beside_v_fma_f32_wavefront_us": {"mfma_alone": round(t_m, 1), "valu_alone": round(t_v, 1),
                                              "together": round(t_both, 1), "sum": round(t_m + t_v, 1)},
            "same_wavefront_1_mfma_16_v_fma_f32_ns_per_mfma_per_simd": round(t_16 * 1e3 / (2 * (m2 // 2) * 16), 3),
            "same_wavefront_1_mfma_16_v_fma_f32_tops": round(cus * 8 * (m2 // 2) * 16 * ops / t_16 / 1e6, 1)}
    out["mfma_forms"] = forms
    return out


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
    ap.add_argument("--no-peaks", action="store_true", help="skip the machine-peak probes")
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
        nproc, usable = host_cores()
        cpu = {"value": round(b / sec / 1e9, 3), "unit": "GB/s", "cores": threads, "nproc": nproc,
               "cpus_usable": usable, "kind": "port",
               "sample": "%d whole-op passes of the same K=%d N=%d M=%d problem (%.2f ms each), CPU oracle, "
                         "two-phase threading" % (reps, K, N, M, sec * 1e3)}

    extra = {"headline": res}
    if not args.no_peaks:
        head = None
        torch.cuda.empty_cache()
        extra["peaks"] = machine_peaks(torch, rq, N * K // 2)
    roofline_m2048 = None
    cpu_m2048 = None
    if not args.no_extra:
        W4A4 = rq.TYPE_W4A4
        shapes = [
            # BASELINE config 1 (the reference's own CPU-runnable case): plain W4A4, no rotation
            ("config1_w4a4_k4096_n1024_m1", 4096, 1024, 1, "normal", 1.0, "hbm", W4A4),
            ("decode_k5120_n5120_m1", 5120, 5120, 1, "outlier_channels", 0.9, "hbm"),
            ("decode_k5120_n5120_m2", 5120, 5120, 2, "outlier_channels", 0.9, "hbm"),
            ("decode_k5120_n5120_m4", 5120, 5120, 4, "outlier_channels", 0.9, "hbm"),
            ("decode_k5120_n5120_m8", 5120, 5120, 8, "outlier_channels", 0.9, "hbm"),
            ("down_k17408_n5120_m1", 17408, 5120, 1, "relu2", 1.0, "hbm"),
            ("down_k17408_n5120_m16", 17408, 5120, 16, "relu2", 1.0, "hbm"),
            ("prefill_k5120_n17408_m64", 5120, 17408, 64, "student_t4", 0.85, "hbm"),
            ("prefill_k5120_n17408_m512", 5120, 17408, 512, "student_t4", 0.85, "mfma"),
            ("prefill_k5120_n17408_m2048", 5120, 17408, 2048, "student_t4", 0.85, "mfma"),
            ("down_k17408_n5120_m2048", 17408, 5120, 2048, "relu2", 1.0, "mfma"),
            # the reference's perf-mode shape (test-backend-ops perf, patch lines 3067-3074)
            ("perf_k5120_n6144_m1", 5120, 6144, 1, "normal", 1.0, "hbm"),
            ("perf_k5120_n6144_m8", 5120, 6144, 8, "normal", 1.0, "hbm"),
            ("perf_k5120_n6144_m16", 5120, 6144, 16, "normal", 1.0, "hbm"),
            ("perf_k5120_n6144_m512", 5120, 6144, 512, "normal", 1.0, "mfma"),
            # the reference's perf mode times both types (patch lines 3067-3074): plain W4A4 on the largest weight
            ("perf_w4a4_k5120_n17408_m1", 5120, 17408, 1, "normal", 1.0, "hbm", W4A4),
            ("perf_w4a4_k5120_n17408_m512", 5120, 17408, 512, "normal", 1.0, "mfma", W4A4),
        ]
        want = [w for w in args.shapes.split(",") if w]
        for name, k, n, m, kind, clip, bound, *rest in shapes:
            if want and name not in want:
                continue
            head = None
            torch.cuda.empty_cache()
            head = Problem(k, n, m, kind, clip, seed=3, type_=rest[0] if rest else None)
            steps = args.steps if m <= 64 else max(20, args.steps // 10)
            extra[name], _, kms = measure(head, steps, min(args.warmup, steps), bound)
            if name == "prefill_k5120_n17408_m2048":
                ops = 2.0 * m * n * k
                roofline_m2048 = {"bound": "mfma", "achieved": round(ops / kms / 1e9, 1), "peak": INT8_PEAK_TOPS,
                                  "unit": "TOP/s", "frac": round(ops / kms / 1e9 / INT8_PEAK_TOPS, 4),
                                  "traffic": profiled_traffic_bytes(GEMM_PROFILE, "traffic_bytes_per_launch_m2048:"),
                                  "kernel": "rq_gemm6_kernel<1, false> (fp6 MFMA; whole tiles and K slices of one launch)"
                                            if os.environ.get("RQ_GEMM_FP6", "1") != "0" else "rq_gemm_kernel (int8 MFMA)",
                                  "kernel_us": round(kms * 1e3, 3), "workload": "W4A4H K=5120 N=17408 M=2048",
                                  "op_us": extra[name]["op_us"], "op_tops": extra[name]["op_tops"],
                                  "op_frac": extra[name]["op_frac_of_int8_peak"]}
                if not args.no_cpu:
                    # the CPU path beside the M = 2048 half of the metric: one whole pass of the oracle, whose result
                    # is also what this problem's GPU output is compared with
                    from oracle import rq_oracle
                    sec, threads, want_y = cpu_one_pass(rq_oracle, head)
                    nproc, usable = host_cores()
                    cpu_m2048 = {"value": round(ops / sec / 1e12, 4), "unit": "TOP/s", "cores": threads, "nproc": nproc,
                                 "cpus_usable": usable, "kind": "port",
                                 "sample": "one whole-op pass of the same K=%d N=%d M=%d problem (%.2f s), CPU oracle, "
                                           "two-phase threading" % (k, n, m, sec),
                                 "parity_vs_oracle": head.check(rq_oracle, want_y)}
                    del want_y

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
                     "frac": round(b / kern_ms / 1e6 / HBM_PEAK_GBS, 4), "traffic": profiled_traffic_bytes(),
                     # one token: rotation, quantizer, product and epilogue are ONE launch, so the dominant kernel
                     # is the whole operator (template arguments: Paley order, groups and remainder items in flight)
                     "kernel": "rq_decode_kernel<20, 10, 4>" if res["activation_kernel_us"] is None
                               else "rq_gemv_kernel<1, 4, 1>",
                     "kernel_us": round(kern_ms * 1e3, 3)},
        "roofline_m2048": roofline_m2048,
        "cpu_baseline": cpu,
        "cpu_baseline_m2048": cpu_m2048,
        "parity_vs_oracle": parity,
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
