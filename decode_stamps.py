#!/usr/bin/env python3
"""Where the time goes inside the one-launch decode kernel: phase timestamps of workgroup 0 (cycle counter of the
compute unit, taken by the first rotate wavefront and the first stream wavefront, kept in registers and written out
when the kernel ends). Needs the instrumented build of the library: `make -C ruquant_amd/csrc stamps`.

    python3 decode_stamps.py [K N]...        (default: the benchmark's one-token shapes)
"""
import ctypes
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
os.environ["RQ_LIB_PATH"] = os.path.join(HERE, "ruquant_amd", "lib", "librq_w4a4_stamps.so")

import torch  # noqa: E402
import ruquant_amd as rq  # noqa: E402
from ruquant_amd import synth  # noqa: E402

ROTATE = ["entry", "row arrived", "Sylvester done, row in LDS", "(LDS passes)", "Paley done", "group ranges",
          "codes in LDS", "stream finished"]
STREAM = ["entry", "flag words requested", "all loads issued", "codes seen", "last group folded", "cells complete"]


def main():
    args = [int(a) for a in sys.argv[1:]]
    shapes = list(zip(args[0::2], args[1::2])) or [(5120, 17408), (5120, 5120), (6144, 5120), (4096, 1024)]
    L = rq.load_library()
    L.rq_w4a4_decode_stamps.restype = ctypes.c_int
    for K, N in shapes:
        blocks = synth.random_weight_blocks(N, K, 0, rq.TYPE_W4A4H, clip=0.9)
        W = rq.W4A4Weight(blocks, rq.TYPE_W4A4H, "cuda:0", keep_blocks=False)
        x = torch.from_numpy(synth.activations("normal", 1, K, 1)).to("cuda:0")
        for _ in range(3):
            rq.mul_mat(W, x)
            torch.cuda.synchronize()
        out = (ctypes.c_ulonglong * 64)()   # [0, 16) rotate wavefront, [32, 48) stream wavefront
        if L.rq_w4a4_decode_stamps(out) != 0:
            raise RuntimeError("rq_w4a4_decode_stamps failed")
        st = list(out)
        print("K=%d N=%d (cycles since the rotate wavefront entered the kernel)" % (K, N))
        for i, name in enumerate(ROTATE):
            print("  rotate wavefront  %-28s %7d" % (name, st[i] - st[0]))
        # the same wavefront, in front of the wait at the end of each stage: what a stage computes and what it waits
        for name, before, after in (("row written to LDS", 8, 2), ("Paley sums written", 9, 4),
                                    ("group ranges computed", 11, 5), ("codes written", 12, 6)):
            if st[before]:
                print("  rotate wavefront  %-28s %7d  (then %d until every rotate wavefront has)"
                      % (name, st[before] - st[0], st[after] - st[before]))
        if st[10]:
            print("  rotate wavefront  %-28s %7d" % ("values of the ranges read", st[10] - st[0]))
        for i, name in enumerate(STREAM):
            print("  stream wavefront  %-28s %7d" % (name, st[32 + i] - st[0]))
        for name, i in (("first barrier passed", 13), ("rows and cells worked out", 14), ("remainder items requested", 15)):
            if st[32 + i]:
                print("  stream wavefront  %-28s %7d" % (name, st[32 + i] - st[0]))
        sys.stdout.flush()


if __name__ == "__main__":
    main()
