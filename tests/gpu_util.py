"""Shared helpers of the GPU parity tests: adversarial inputs in the style of the reference's
test-backend-ops initializer (patch lines 2956-2999) and the bit-exact comparison."""
import numpy as np
import torch

import ruquant_amd as rq


def bits_equal(a, b):
    a = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    b = np.ascontiguousarray(b, dtype=np.float32).view(np.uint32)
    return a.shape == b.shape and bool((a == b).all())


def first_mismatch(a, b):
    a32 = np.ascontiguousarray(a, dtype=np.float32)
    b32 = np.ascontiguousarray(b, dtype=np.float32)
    bad = np.argwhere(a32.view(np.uint32) != b32.view(np.uint32))
    if bad.size == 0:
        return "equal"
    i = tuple(bad[0])
    return "%d of %d differ; first at %s: got %r (%08x) want %r (%08x)" % (
        len(bad), a32.size, i, float(a32[i]), int(a32.view(np.uint32)[i]), float(b32[i]), int(b32.view(np.uint32)[i]))


def adversarial_weights(oracle, N, K, type_, seed=1234, wgroup=0, n_rot=None):
    """Float weights whose 64-wide groups differ in scale (x1/4 .. x4), every 7th row flat +-1, quantized with
    the reference's weight-side quantizer. Returns (blocks, float weights)."""
    rng = np.random.default_rng(seed)
    v = rng.uniform(-1.0, 1.0, size=(N, K)).astype(np.float32)
    r = np.arange(N)[:, None]
    i = np.arange(K)[None, :]
    w = v * np.exp2(((i // 64 + r) % 5 - 2).astype(np.float32))
    flat = (np.arange(N) % 7 == 0)
    w[flat] = np.where(v[flat] < 0, -1.0, 1.0)
    w = w.astype(np.float32)
    had = type_ == rq.TYPE_W4A4H
    blocks = oracle.quantize_rows_w(w, hadamard=had, n_rot=n_rot or K, wgroup=wgroup)
    return blocks, w


def adversarial_activations(M, K, type_, w_float, seed=99):
    """uniform(-1,1) scaled per 64-wide group (x1/8 .. x8) and per token (x1/2, 1, 2); for W4A4 every 5th token
    takes the signs of weight row 0 (an aligned flat row, the case that stresses the int32 total)."""
    rng = np.random.default_rng(seed)
    x = rng.uniform(-1.0, 1.0, size=(M, K)).astype(np.float32)
    r = np.arange(M)[:, None]
    i = np.arange(K)[None, :]
    x = x * np.exp2(((i // 64) % 7 - 3).astype(np.float32) + (r % 3 - 1).astype(np.float32))
    if type_ == rq.TYPE_W4A4:
        aligned = (np.arange(M) % 5 == 0)
        x[aligned] = np.where(w_float[0] < 0, -1.0, 1.0)[None, :]
    return x.astype(np.float32)


def run_gpu(weight, x_np):
    x = torch.from_numpy(x_np).to(weight.device)
    y = rq.mul_mat(weight, x)
    torch.cuda.synchronize()
    return y.cpu().numpy()
