"""Runs in a process of its own, started by test_gpu_variants.py with RQ_DECODE_FUSED=0: one token through the
rotation kernel + GEMV instead of the one-launch decode kernel, against the oracle. Prints `ALL OK`."""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)

import ruquant_amd as rq  # noqa: E402
from oracle import rq_oracle  # noqa: E402
from gpu_util import adversarial_weights, adversarial_activations, bits_equal, first_mismatch, run_gpu  # noqa: E402

assert os.environ.get("RQ_DECODE_FUSED") == "0"
bad = 0
for type_, N, K, wgroup in ((rq.TYPE_W4A4H, 1000, 5120, 0), (rq.TYPE_W4A4H, 320, 6144, 64), (rq.TYPE_W4A4, 136, 4096, 256),
                            (rq.TYPE_W4A4H, 192, 1536, 0)):
    blocks, wf = adversarial_weights(rq_oracle, N, K, type_, wgroup=wgroup)
    W = rq.W4A4Weight(blocks, type_, "cuda:0")
    x = adversarial_activations(1, K, type_, wf, seed=5)
    got = run_gpu(W, x)
    want = rq_oracle.mul_mat(type_, blocks, x, W.clip, n_rot=max(W.n_rot, 0))
    ok = bits_equal(got, want)
    print("type=%d N=%d K=%d wgroup=%d: %s" % (type_, N, K, wgroup, "ok" if ok else first_mismatch(got, want)), flush=True)
    bad += not ok
print("ALL OK" if bad == 0 else "%d FAILED" % bad, flush=True)
sys.exit(1 if bad else 0)
