"""Runs in a process of its own, started by test_gpu_act_group.py with RQ_ACT_GROUP set (the library reads the
variable once per process, as the reference does): the op and the activation quantizer with activation groups of
128 or 256 against the oracle with the same group width, bit for bit. Prints one line per case and `ALL OK`."""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)

import ruquant_amd as rq  # noqa: E402
from oracle import rq_oracle  # noqa: E402
from gpu_util import adversarial_weights, adversarial_activations, bits_equal, first_mismatch, run_gpu  # noqa: E402

G = int(os.environ["RQ_ACT_GROUP"])
assert rq.load_library().rq_w4a4_act_group() == G
DEV = "cuda:0"
bad = 0
cases = [(rq.TYPE_W4A4H, 200, 1536, 0), (rq.TYPE_W4A4H, 200, 1536, 64), (rq.TYPE_W4A4, 136, 1024, 256),
         (rq.TYPE_W4A4H, 256, 5120, 0), (rq.TYPE_W4A4H, 320, 768, 64), (rq.TYPE_W4A4H, 128, 17408, 0)]
for type_, N, K, wgroup in cases:
    blocks, wf = adversarial_weights(rq_oracle, N, K, type_, wgroup=wgroup)
    if wgroup == 64:
        # weight groups of 64 need activation groups of 64: the reference asserts (patch lines 169-170), this refuses
        try:
            rq.W4A4Weight(blocks, type_, DEV)
            print("wgroup=64 with RQ_ACT_GROUP=%d was not refused" % G, flush=True)
            bad += 1
        except rq.RqError as e:
            print("wgroup=64 refused: %s" % e, flush=True)
        continue
    W = rq.W4A4Weight(blocks, type_, DEV)
    # up to four tokens the GEMV folds the wide groups, from five to 64 the skinny MFMA kernel (one or two token tiles
    # per wavefront, blocks of 32 tokens), beyond that the fp6 GEMM, whose MFMAs of a group chain through the accumulator
    for M in (1, 2, 3, 5, 8, 9, 16, 17, 32, 33, 40, 64, 65, 130, 300):
        x = adversarial_activations(M, K, type_, wf, seed=M)
        got = run_gpu(W, x)
        want = rq_oracle.mul_mat(type_, blocks, x, W.clip, n_rot=max(W.n_rot, 0), G=G)
        ok = bits_equal(got, want)
        print("mul_mat type=%d N=%d K=%d wgroup=%d M=%d: %s" % (type_, N, K, wgroup, M,
                                                                "ok" if ok else first_mismatch(got, want)), flush=True)
        bad += not ok
# the reference's own shape list (test-backend-ops, patch lines 3024-3040), both types
from test_gpu_parity import _shapes_reference  # noqa: E402
last = None
for N, M, K in sorted(_shapes_reference(), key=lambda s: (s[0], s[2], s[1])):
    for type_ in (rq.TYPE_W4A4, rq.TYPE_W4A4H):
        if K % G != 0:
            continue
        if last is None or last[0] != (N, K, type_):
            blocks, wf = adversarial_weights(rq_oracle, N, K, type_)
            last = ((N, K, type_), blocks, wf, rq.W4A4Weight(blocks, type_, DEV))
        _, blocks, wf, W = last
        x = adversarial_activations(M, K, type_, wf, seed=M)
        got = run_gpu(W, x)
        want = rq_oracle.mul_mat(type_, blocks, x, W.clip, n_rot=max(W.n_rot, 0), G=G)
        ok = bits_equal(got, want)
        if not ok:
            print("reference shape type=%d N=%d M=%d K=%d: %s" % (type_, N, M, K, first_mismatch(got, want)), flush=True)
        bad += not ok
print("reference shapes done", flush=True)
for K, had in ((1536, True), (5120, True), (1024, False)):
    rng = np.random.default_rng(K)
    x = (rng.standard_normal((3, K)) * np.exp2(rng.integers(-3, 4, size=(3, K // 64)).repeat(64, axis=1))).astype(np.float32)
    got = rq.quantize_act(torch.from_numpy(x).to(DEV), 0.9, hadamard_=had)
    for t in range(3):
        want = rq_oracle.quantize_row_a4h(x[t], 0.9, K, G) if had else rq_oracle.quantize_row_a(x[t], 0.9, G)
        ok = got[t].tobytes() == want.tobytes()
        print("quantize_act K=%d hadamard=%s token %d: %s" % (K, had, t, "ok" if ok else "MISMATCH"), flush=True)
        bad += not ok
print("ALL OK" if bad == 0 else "%d FAILED" % bad, flush=True)
sys.exit(1 if bad else 0)
