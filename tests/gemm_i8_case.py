"""Runs in a process of its own, started by test_gpu_gemm6.py with RQ_GEMM_FP6=0 (read once per process): prepared
weights then carry no fp6 plane and wide batches run on the int8 MFMA kernel (wide, narrow and half tiles, the skinny
tail), against the oracle, bit for bit. Prints one line per case and `ALL OK`."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)

import ruquant_amd as rq  # noqa: E402
from oracle import rq_oracle  # noqa: E402
from gpu_util import adversarial_weights, adversarial_activations, bits_equal, first_mismatch, run_gpu  # noqa: E402

assert os.environ.get("RQ_GEMM_FP6") == "0"
DEV = "cuda:0"
L = rq.load_library()
# no fp6 plane: codes, scales, multipliers and the flag word only
assert L.rq_w4a4_prepared_bytes(5120, 1024) < 1024 * 5120 // 2 + 1024 * 5120 // 64 + 4 * 1024 + 4096
bad = 0
cases = [  # (type, N, K, M, weight group)
    (rq.TYPE_W4A4H, 6144, 1024, 512, 0), (rq.TYPE_W4A4H, 6100, 1536, 500, 0), (rq.TYPE_W4A4, 6144, 1024, 450, 256),
    (rq.TYPE_W4A4H, 6144, 768, 512, 64),            # half tiles
    (rq.TYPE_W4A4H, 8300, 256, 1024, 0), (rq.TYPE_W4A4H, 16500, 256, 520, 64),   # whole wide rounds + a tail
    (rq.TYPE_W4A4H, 256, 6144, 65, 0), (rq.TYPE_W4A4, 256, 6144, 130, 0), (rq.TYPE_W4A4H, 136, 5120, 200, 0),
    (rq.TYPE_W4A4H, 2048, 5120, 2048, 0),           # 128 wide tiles
]
for type_, N, K, M, wgroup in cases:
    blocks, wf = adversarial_weights(rq_oracle, N, K, type_, wgroup=wgroup)
    W = rq.W4A4Weight(blocks, type_, DEV)
    x = adversarial_activations(M, K, type_, wf, seed=M)
    got = run_gpu(W, x)
    want = rq_oracle.mul_mat(type_, blocks, x, W.clip, n_rot=max(W.n_rot, 0))
    ok = bits_equal(got, want)
    print("type=%d N=%d K=%d M=%d wgroup=%d: %s" % (type_, N, K, M, wgroup, "ok" if ok else first_mismatch(got, want)),
          flush=True)
    bad += not ok
print("ALL OK" if bad == 0 else "%d FAILED" % bad, flush=True)
sys.exit(1 if bad else 0)
