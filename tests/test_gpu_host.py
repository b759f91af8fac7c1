"""The C++ host over the ggml-style adapter (the counterpart of the reference's Rust host): first use, steady state
and fusion through the reference's own entry-point names, compared bit for bit with the oracle."""
import json
import os
import subprocess

import numpy as np
import pytest

import ruquant_amd as rq
from ruquant_amd import synth
from tests.gpu_util import bits_equal, first_mismatch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "ruquant_amd", "lib", "rq_host")


def test_host_binary_is_built_and_prints_usage():
    assert os.path.exists(HOST), "build it with make -C ruquant_amd/csrc"
    r = subprocess.run([HOST], capture_output=True, text=True)
    assert r.returncode == 2 and "usage" in r.stderr


def _run(tmp_path, type_, K, N, M, blocks, x, extra=()):
    blocks.tofile(tmp_path / "w.bin")
    x.tofile(tmp_path / "x.bin")
    cmd = [HOST, str(type_), str(K), str(N), str(M), str(tmp_path / "w.bin"), str(tmp_path / "x.bin"),
           str(tmp_path / "y.bin"), "3"] + [str(e) for e in extra]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
    return r, (np.fromfile(tmp_path / "y.bin", dtype=np.float32).reshape(M, N) if r.returncode == 0 else None)


@pytest.mark.gpu
@pytest.mark.parametrize("type_,K,N,M,clip", [(rq.TYPE_W4A4H, 5120, 1024, 8, 0.9), (rq.TYPE_W4A4, 1536, 200, 3, 0.0),
                                                (rq.TYPE_W4A4H, 6144, 512, 70, 0.0)])
def test_host_matches_oracle(oracle, tmp_path, type_, K, N, M, clip):
    blocks = synth.random_weight_blocks(N, K, 21, type_, clip=clip)
    x = synth.activations("student_t4", M, K, 22)
    r, y = _run(tmp_path, type_, K, N, M, blocks, x)
    assert r.returncode == 0, r.stderr
    info = json.loads(r.stdout.strip().splitlines()[-1])
    assert info["supported"] and not info["ready_before"] and info["ready_after"]
    want = oracle.mul_mat(type_, blocks, x, float(np.float32(clip)) if clip else 1.0, n_rot=K if type_ == rq.TYPE_W4A4H else 0)
    assert bits_equal(y, want), first_mismatch(y, want)


@pytest.mark.gpu
def test_host_fuses_two_weights_of_one_input(oracle, tmp_path):
    type_, K, N, N2, M = rq.TYPE_W4A4H, 5120, 640, 256, 4
    b1 = synth.random_weight_blocks(N, K, 31, type_, clip=0.9)
    b2 = synth.random_weight_blocks(N2, K, 32, type_, clip=0.9)
    x = synth.activations("outlier_channels", M, K, 33)
    b2.tofile(tmp_path / "w2.bin")
    r, y = _run(tmp_path, type_, K, N, M, b1, x, extra=("fuse", tmp_path / "w2.bin", N2, tmp_path / "y2.bin"))
    assert r.returncode == 0, r.stderr
    info = json.loads(r.stdout.strip().splitlines()[-1])
    assert info["fused"]
    y2 = np.fromfile(tmp_path / "y2.bin", dtype=np.float32).reshape(M, N2)
    c = float(np.float32(0.9))
    assert bits_equal(y, oracle.mul_mat(type_, b1, x, c, n_rot=K))
    assert bits_equal(y2, oracle.mul_mat(type_, b2, x, c, n_rot=K))


@pytest.mark.gpu
@pytest.mark.parametrize("M", [2, 16, 70])
def test_host_shares_the_quantized_activation_between_separate_calls(oracle, tmp_path, M):
    """Two MUL_MATs of one x as separate calls inside one graph evaluation (the reference's rq_act_cache, patch lines
    2160-2172): the second is a hit and still bit-identical; after x changed in place and a new evaluation began, the
    first call is a miss again and both results are those of the new x."""
    type_, K, N, N2 = rq.TYPE_W4A4H, 5120, 640, 256
    b1 = synth.random_weight_blocks(N, K, 41, type_, clip=0.9)
    b2 = synth.random_weight_blocks(N2, K, 42, type_, clip=0.9)
    x = synth.activations("outlier_channels", M, K, 43)
    b2.tofile(tmp_path / "w2.bin")
    r, y = _run(tmp_path, type_, K, N, M, b1, x, extra=("cache", tmp_path / "w2.bin", N2, tmp_path / "y2.bin"))
    assert r.returncode == 0, r.stderr
    info = json.loads(r.stdout.strip().splitlines()[-1])
    assert (info["act_hits_first"], info["act_misses_first"]) == (1, 1)
    assert (info["act_hits_again"], info["act_misses_again"]) == (1, 1)
    c = float(np.float32(0.9))
    y2_first = np.fromfile(str(tmp_path / "y2.bin") + ".first", dtype=np.float32).reshape(M, N2)
    assert bits_equal(y2_first, oracle.mul_mat(type_, b2, x, c, n_rot=K)), "hit differs from a fresh transform"
    y2 = np.fromfile(tmp_path / "y2.bin", dtype=np.float32).reshape(M, N2)
    assert bits_equal(y, oracle.mul_mat(type_, b1, -x, c, n_rot=K)), "stale activation after graph_begin"
    assert bits_equal(y2, oracle.mul_mat(type_, b2, -x, c, n_rot=K))


@pytest.mark.gpu
def test_host_reports_unsupported_shape(tmp_path):
    # K with no Hadamard factorization: the backend declines, ggml would fall back to the CPU
    type_, K, N, M = rq.TYPE_W4A4H, 7 * 256, 64, 1
    blocks = synth.random_weight_blocks(N, K, 1, type_)
    x = synth.activations("normal", M, K, 2)
    r, _ = _run(tmp_path, type_, K, N, M, blocks, x)
    assert r.returncode == 3 and json.loads(r.stdout.strip())["supported"] is False
