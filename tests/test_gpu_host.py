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


def _run(tmp_path, type_, K, N, M, blocks, x, extra=(), env=None):
    blocks.tofile(tmp_path / "w.bin")
    x.tofile(tmp_path / "x.bin")
    cmd = [HOST, str(type_), str(K), str(N), str(M), str(tmp_path / "w.bin"), str(tmp_path / "x.bin"),
           str(tmp_path / "y.bin"), "3"] + [str(e) for e in extra]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=120, env=env)
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


@pytest.mark.gpu
def test_python_shared_activation_layer_chain(oracle):
    """SharedActivation (the Python host's counterpart of the reference's rq_act_cache, patch lines 1996-2023,
    2163-2172) over one transformer layer's seven products in the layer's dataflow: q, k, v share one quantized x,
    gate and up another. Every output equals the oracle's bits; hits and misses are counted. Orders in which the
    second weight of a shared x is the larger one (k before q, up after a smaller gate stand-in) must miss again
    where the split-K cells of the first call do not cover its rows."""
    import numpy as np
    import torch
    import ruquant_amd as rq
    from ruquant_amd import synth
    from tests.gpu_util import bits_equal, first_mismatch

    dev = "cuda:0"
    type_ = rq.TYPE_W4A4H
    shapes = {"q": (5120, 1536), "k": (5120, 256), "v": (5120, 256), "o": (1536, 5120), "gate": (5120, 2176),
              "up": (5120, 2176), "down": (2176 * 2, 5120)}
    shapes["down"] = (4352, 5120)     # 68 x 64: the long Paley stage
    shapes["gate"] = shapes["up"] = (5120, 4352)
    blocks = {n: synth.random_weight_blocks(N, K, 50 + i, type_, clip=0.0) for i, (n, (K, N)) in enumerate(shapes.items())}
    W = {n: rq.W4A4Weight(blocks[n], type_, dev) for n in shapes}
    L = rq.load_library()
    for M in (1, 3, 16, 40, 70):
        x0 = synth.activations("normal", M, 5120, 60 + M)
        ws = torch.empty(max(L.rq_w4a4_workspace_bytes(type_, K, N, M) for K, N in shapes.values()), dtype=torch.uint8,
                         device=dev)
        sa = rq.SharedActivation(ws)
        out = {n: torch.full((M, N), float("nan"), dtype=torch.float32, device=dev) for n, (K, N) in shapes.items()}
        xd = torch.from_numpy(x0).to(dev)
        for order in (("q", "k", "v"), ("k", "q", "v")):
            sa.begin()
            h0, m0 = sa.hits, sa.misses
            for n in order:
                sa.mul_mat(W[n], xd, out[n])
            # one miss for the first weight; a later, larger weight misses again when the cells cleared for the first
            # do not cover its rows (k before q), everything else hits
            expect_miss = 1 if order[0] == "q" else 2
            assert (sa.misses - m0, sa.hits - h0) == (expect_miss, 3 - expect_miss), (M, order, sa.misses - m0)
            torch.cuda.synchronize()
            ref = {n: oracle.mul_mat(type_, blocks[n], x0, 1.0, n_rot=5120) for n in ("q", "k", "v")}
            for n in order:
                got = out[n].cpu().numpy()
                assert bits_equal(got, ref[n]), "M=%d order=%s %s: %s" % (M, order, n, first_mismatch(got, ref[n]))
        sa.mul_mat(W["o"], out["q"], out["o"])
        sa.mul_mat(W["gate"], out["o"], out["gate"])
        sa.mul_mat(W["up"], out["o"], out["up"])
        sa.mul_mat(W["down"], out["up"], out["down"])
        torch.cuda.synchronize()
        ro = oracle.mul_mat(type_, blocks["o"], ref["q"], 1.0, n_rot=1536)
        rg = oracle.mul_mat(type_, blocks["gate"], ro, 1.0, n_rot=5120)
        ru = oracle.mul_mat(type_, blocks["up"], ro, 1.0, n_rot=5120)
        rd = oracle.mul_mat(type_, blocks["down"], ru, 1.0, n_rot=4352)
        for n, r in (("o", ro), ("gate", rg), ("up", ru), ("down", rd)):
            got = out[n].cpu().numpy()
            assert bits_equal(got, r), "M=%d %s: %s" % (M, n, first_mismatch(got, r))


@pytest.mark.gpu
@pytest.mark.parametrize("M", [1, 8, 200])
def test_host_keeps_one_copy_of_the_codes(oracle, tmp_path, M):
    """First use through the adapter rewrites the weight's own buffer (the reference's in-place repack, patch lines
    2046-2075): beside the tensor only the fp6 plane of the wide-batch kernel stays resident, not a second copy of the
    codes, and the results are the oracle's bits. With RQ_HOST_IN_PLACE=0 the prepared weight is a buffer of its own
    (the tensor stays readable as blocks) and the same bits come out."""
    type_, K, N = rq.TYPE_W4A4H, 5120, 4096
    blocks = synth.random_weight_blocks(N, K, 41, type_, clip=0.9)
    x = synth.activations("student_t4", M, K, 42)
    want = oracle.mul_mat(type_, blocks, x, float(np.float32(0.9)), n_rot=K)
    info = {}
    for in_place in (1, 0):
        env = dict(os.environ)
        env["RQ_HOST_IN_PLACE"] = str(in_place)
        # (a second weight of the same shape goes first, so that the scratch buffer has its size when the memory
        # around the first use of the weight under test is read)
        blocks.tofile(tmp_path / "w2.bin")
        r, y = _run(tmp_path, type_, K, N, M, blocks, x, extra=("fuse", tmp_path / "w2.bin", N, tmp_path / "y2.bin"), env=env)
        assert r.returncode == 0, r.stderr
        info[in_place] = json.loads(r.stdout.strip().splitlines()[-1])
        assert info[in_place]["in_place"] == bool(in_place)
        assert bits_equal(y, want), "in_place=%d: %s" % (in_place, first_mismatch(y, want))
    slack = 4 << 20                       # the allocator's granularity
    a, b = info[1], info[0]
    assert a["tensor_bytes"] == N * (K // 256) * 144
    assert abs(a["first_use_bytes_beside_tensor"] - a["plane6_bytes"]) <= slack, a
    assert abs(b["first_use_bytes_beside_tensor"] - b["prepared_bytes"]) <= slack, b
    # in place: nothing of the size of the codes (N K / 2) is held twice
    assert a["first_use_bytes_beside_tensor"] <= b["first_use_bytes_beside_tensor"] - N * K // 2 + slack


@pytest.mark.gpu
def test_prepare_in_place_python_binding(oracle):
    """rq_w4a4_prepare_inplace through the Python binding over the token counts of every product kernel, ragged row
    counts, weight multipliers and a long row; a shape too small to hold its prepared form in place is refused."""
    import torch
    dev = "cuda:0"
    from tests.gpu_util import adversarial_weights, adversarial_activations, run_gpu
    for type_, N, K, wgroup in ((rq.TYPE_W4A4H, 1000, 5120, 0), (rq.TYPE_W4A4, 777, 1024, 64),
                                (rq.TYPE_W4A4H, 320, 17408, 256), (rq.TYPE_W4A4H, 4100, 256, 0)):
        blocks, wf = adversarial_weights(oracle, N, K, type_, wgroup=wgroup)
        W = rq.W4A4Weight(blocks, type_, dev, in_place=True)
        assert W.blocks is None and W.prepared.numel() == blocks.nbytes
        for M in (1, 3, 16, 70, 300):
            x = adversarial_activations(M, K, type_, wf, seed=M)
            got = run_gpu(W, x)
            want = oracle.mul_mat(type_, blocks, x, W.clip, n_rot=max(W.n_rot, 0))
            assert bits_equal(got, want), "N=%d K=%d M=%d: %s" % (N, K, M, first_mismatch(got, want))
    L = rq.load_library()
    tiny = torch.zeros(4096, dtype=torch.uint8, device=dev)
    stage = torch.zeros(L.rq_w4a4_inplace_staging_bytes(256, 3), dtype=torch.uint8, device=dev)
    n6 = L.rq_w4a4_plane6_bytes(256, 3)
    p6 = torch.zeros(max(n6, 256), dtype=torch.uint8, device=dev)
    # three rows of one block each: 432 bytes of blocks cannot hold a panel of 64 padded rows
    rc = L.rq_w4a4_prepare_inplace(tiny.data_ptr(), 256, 3, p6.data_ptr(), n6, stage.data_ptr(), stage.numel(), None)
    assert rc == -2
    torch.cuda.synchronize()
