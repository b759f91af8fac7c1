"""Format variants over the reference's own shape lists (test-backend-ops, patches/llama.cpp-ruquant.patch lines
3024-3040, re-run there under RQ_WGROUP and RQ_ROT_BLOCKS; patches/mx-llama.cpp-ruquant.patch lines 6468-6474 for the
shapes of one GPU of four): weight multipliers per block and per 64 inputs, block-diagonal rotations of K / 2, K / 4
and K / 8, all against the CPU oracle at zero tolerance. The reference selects the variants through the environment
of its quantizer; here they are arguments of the weight quantizer, so the cases run in this process. Activation
groups of 128 / 256 and the clip taken from the environment are process-wide switches of the library and run in
child processes (test_gpu_act_group.py, test_env_clip_reaches_the_kernels below)."""
import os
import subprocess
import sys

import numpy as np
import pytest

import ruquant_amd as rq
from tests.gpu_util import bits_equal, first_mismatch, adversarial_weights, adversarial_activations, run_gpu
from tests.test_gpu_parity import _shapes_reference

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HERE = os.path.dirname(os.path.abspath(__file__))

_W = {}


def _weights(oracle, N, K, type_, wgroup, n_rot):
    key = (N, K, type_, wgroup, n_rot)
    if key not in _W:
        blocks, wf = adversarial_weights(oracle, N, K, type_, wgroup=wgroup, n_rot=n_rot)
        _W.clear()
        _W[key] = (blocks, wf, rq.W4A4Weight(blocks, type_, DEV))
    return _W[key]


def _check(oracle, type_, N, M, K, wgroup=0, n_rot=None):
    blocks, wf, W = _weights(oracle, N, K, type_, wgroup, n_rot)
    x = adversarial_activations(M, K, type_, wf, seed=7 * M + 1)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, blocks, x, W.clip, n_rot=max(W.n_rot, 0))
    assert bits_equal(got, want), first_mismatch(got, want)


SHAPES = sorted(_shapes_reference(), key=lambda s: (s[0], s[2], s[1]))
# the shapes of one GPU of four (narrow-K Hadamards: 4352 = 68 x 64, 1536 = 12 x 128)
MX_SHAPES = [(n, m, k) for m in (1, 8, 16) for (n, k) in ((4096, 5120), (8704, 5120), (5120, 4352), (5120, 1536))]


# (the decorator on top varies fastest: the token counts of one weight run back to back and share its quantization)
@pytest.mark.parametrize("N,M,K", sorted(MX_SHAPES, key=lambda s: (s[0], s[2], s[1])), ids=lambda v: str(v))
@pytest.mark.parametrize("type_", [rq.TYPE_W4A4, rq.TYPE_W4A4H], ids=["w4a4", "w4a4h"])
def test_shapes_of_one_gpu_of_four(oracle, type_, N, M, K):
    _check(oracle, type_, N, M, K)


@pytest.mark.parametrize("N,M,K", SHAPES, ids=lambda v: str(v))
@pytest.mark.parametrize("wgroup", [256, 64])
@pytest.mark.parametrize("type_", [rq.TYPE_W4A4, rq.TYPE_W4A4H], ids=["w4a4", "w4a4h"])
def test_reference_shapes_with_weight_groups(oracle, type_, wgroup, N, M, K):
    """RQ_WGROUP=1 (a multiplier per block of 256) and RQ_WGROUP=64 (per 64 inputs), reference lines 2531-2538."""
    _check(oracle, type_, N, M, K, wgroup=wgroup)


@pytest.mark.parametrize("N,M,K", SHAPES, ids=lambda v: str(v))
@pytest.mark.parametrize("blocks", [2, 4, 8])
def test_reference_shapes_with_rotation_blocks(oracle, blocks, N, M, K):
    """RQ_ROT_BLOCKS = 2 / 4 / 8 (reference lines 2687-2694): block-diagonal Hadamards of K / blocks."""
    _check(oracle, rq.TYPE_W4A4H, N, M, K, n_rot=K // blocks)


def _child(script, env_extra, timeout=600):
    env = dict(os.environ)
    env.update(env_extra)
    out = subprocess.run([sys.executable, "-u", os.path.join(HERE, script)], env=env, capture_output=True, text=True,
                         timeout=timeout)
    assert out.returncode == 0 and "ALL OK" in out.stdout, out.stdout[-3000:] + out.stderr[-2000:]
    return out.stdout


def test_env_clip_reaches_the_kernels():
    """RQ_ACT_CLIP_H=0.85 with no clip in the tensor (benchmark configuration 3): the clip travels from the
    environment through rq_w4a4_resolve_clip into the kernels."""
    out = _child("env_clip_case.py", {"RQ_ACT_CLIP_H": "0.85"})
    assert "clip=0.85" in out


def test_one_token_through_the_two_launch_path():
    """RQ_DECODE_FUSED=0, the library's one debug switch: one token takes the rotation kernel + GEMV that serve two
    and three tokens instead of the one-launch kernel; same bits."""
    _child("decode_two_launch_case.py", {"RQ_DECODE_FUSED": "0"})
