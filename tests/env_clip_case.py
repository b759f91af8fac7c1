"""Runs in a process of its own, started by test_gpu_variants.py with RQ_ACT_CLIP_H=0.85 (the library reads the
variable once per process, as the reference does, patch lines 2590-2600): benchmark configuration 3 (W4A4H, K = 5120,
N = 17408, Student-t activations, no clip in the tensor) with the clip that rq_w4a4_resolve_clip returns, against the
oracle given 0.85 explicitly. Prints `ALL OK`."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)

import ruquant_amd as rq  # noqa: E402
from ruquant_amd import synth  # noqa: E402
from oracle import rq_oracle  # noqa: E402
from gpu_util import bits_equal, first_mismatch, run_gpu  # noqa: E402

assert os.environ.get("RQ_ACT_CLIP_H") == "0.85"
K, N = 5120, 17408
blocks = synth.random_weight_blocks(N, K, 3, rq.TYPE_W4A4H, clip=0.0)      # pad[1] = 0: no clip in the tensor
W = rq.W4A4Weight(blocks, rq.TYPE_W4A4H, "cuda:0")
want_clip = float(np.float32(0.85))
print("clip=%.2f" % W.clip, flush=True)
bad = W.clip != want_clip
# the W4A4 variable is not set: a W4A4 tensor keeps clip 1
W0 = rq.W4A4Weight(synth.random_weight_blocks(64, 256, 1, rq.TYPE_W4A4), rq.TYPE_W4A4, "cuda:0")
bad |= W0.clip != 1.0
for M in (1, 64, 512, 2048):   # (the last is benchmark configuration 3 at its full size: about a second of oracle)
    x = synth.activations("student_t4", M, K, 3)
    got = run_gpu(W, x)                                                      # the op takes W.clip, i.e. the environment's
    want = rq_oracle.mul_mat(rq.TYPE_W4A4H, blocks, x, want_clip, n_rot=K)
    ok = bits_equal(got, want)
    print("M=%d: %s" % (M, "ok" if ok else first_mismatch(got, want)), flush=True)
    bad |= not ok
print("ALL OK" if not bad else "FAILED", flush=True)
sys.exit(1 if bad else 0)
