"""GPU parity on seeded random problems: row lengths with every kind of rotation the type admits (Paley factors 1,
12, 20, 28, 44, 60, 68 times a power of two, whole-row and block-diagonal), ragged row counts, token counts on both
sides of every switch of the dispatcher (GEMV / skinny MFMA / tiled GEMM, one or two token blocks, leftover tiles),
legacy and grouped weight multipliers. Zero tolerance against the CPU oracle."""
import numpy as np
import pytest

import ruquant_amd as rq
from tests.gpu_util import bits_equal, first_mismatch, adversarial_weights, adversarial_activations, run_gpu

pytestmark = pytest.mark.gpu

DEV = "cuda:0"

# K = p * 2^j * (blocks of the rotation): all multiples of 256 with a Paley x Sylvester factorization
ROW_LENGTHS = [256, 512, 768, 1024, 1280, 1536, 1792, 2048, 2816, 3072, 3840, 4352, 5120, 6144, 7168, 8192]
TOKENS = [1, 2, 3, 4, 5, 7, 8, 9, 16, 17, 31, 32, 33, 40, 41, 63, 64, 65, 96, 127, 128, 129, 200, 257]


def _cases():
    rng = np.random.default_rng(20261125)
    out = []
    for i in range(48):
        K = int(rng.choice(ROW_LENGTHS))
        type_ = rq.TYPE_W4A4H if i % 3 else rq.TYPE_W4A4
        N = int(rng.integers(1, 520))
        M = int(TOKENS[i % len(TOKENS)])
        wgroup = int(rng.choice([0, 0, 256, 64]))
        n_rot = K
        if type_ == rq.TYPE_W4A4H and rng.uniform() < 0.3:
            # a block-diagonal rotation: a divisor of K that is itself a multiple of 256 and factorizes
            for d in (2, 3, 4, 5, 7):
                if K % d == 0 and (K // d) % 256 == 0 and rq.hadamard_factor(K // d) is not None:
                    n_rot = K // d
                    break
        if type_ == rq.TYPE_W4A4H and rq.hadamard_factor(n_rot) is None:
            type_ = rq.TYPE_W4A4
        out.append((i, type_, N, K, M, wgroup, n_rot))
    return out


@pytest.mark.parametrize("case", _cases(), ids=lambda c: "%d_t%d_n%d_k%d_m%d_g%d_r%d" % c)
def test_random_problem(oracle, case):
    i, type_, N, K, M, wgroup, n_rot = case
    had = type_ == rq.TYPE_W4A4H
    blocks, wf = adversarial_weights(oracle, N, K, type_, seed=1000 + i, wgroup=wgroup, n_rot=n_rot if had else None)
    W = rq.W4A4Weight(blocks, type_, DEV)
    if had:
        assert W.n_rot == n_rot
    x = adversarial_activations(M, K, type_, wf, seed=2000 + i)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, blocks, x, W.clip, n_rot=n_rot if had else 0)
    assert bits_equal(got, want), first_mismatch(got, want)
