"""The wide-batch product kernel on the fp6 MFMA (rq_gemm6.hip): launches made of whole tiles and of tiles cut along
K, compared bit for bit with the oracle; and the int8 MFMA kernel it replaced, which RQ_GEMM_FP6=0 still selects, in a
child process (the variable is read once per process)."""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import ruquant_amd as rq
from ruquant_amd import synth
from tests.gpu_util import adversarial_weights, adversarial_activations, bits_equal, first_mismatch, run_gpu

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HERE = os.path.dirname(os.path.abspath(__file__))


def test_prepared_weight_carries_the_fp6_plane():
    L = rq.load_library()
    K, N = 5120, 1000
    compact = N * K // 2
    # padded to row tiles of 256: 1024 rows x 0.75 bytes per weight
    assert L.rq_w4a4_prepared_bytes(K, N) >= compact + 1024 * K * 3 // 4


@pytest.mark.parametrize("type_,wgroup", [(rq.TYPE_W4A4H, 0), (rq.TYPE_W4A4, 64), (rq.TYPE_W4A4, 256)],
                         ids=["w4a4h", "w4a4_wgroup64", "w4a4_wgroup256"])
def test_leftover_tiles_cut_along_k_uneven_slices(oracle, type_, wgroup):
    """8 row tiles x 33 token tiles = 264 tiles: 256 run whole, the last 8 (one row tile, eight token tiles) are cut
    into five slices of 6 or 7 steps of the row's 34 (K = 4352 = 68 x 64: an odd step count in most slices), which
    meet through their slabs. Ragged rows and tokens, with and without weight multipliers."""
    N, K, M = 2000, 4352, 4200
    blocks, wf = adversarial_weights(oracle, N, K, type_, wgroup=wgroup)
    W = rq.W4A4Weight(blocks, type_, DEV)
    x = adversarial_activations(M, K, type_, wf, seed=7)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, blocks, x, W.clip, n_rot=max(W.n_rot, 0))
    assert bits_equal(got, want), first_mismatch(got, want)
    # twice on the same workspace: the arrival counters are left zero
    got2 = run_gpu(W, x)
    assert bits_equal(got2, want), first_mismatch(got2, want)


def test_slices_longest_row_extreme_sums(oracle):
    """K = 32768 with every tile cut along K (1 row tile x 12 token tiles: 13 slices of 19 or 20 steps each), inputs
    that drive the sums to their ends: rows of all -8 / all +7 codes against tokens that quantize to q - z = +-15 with
    m = 255 in all 512 groups. Within a slice the biased fp32 accumulator moves by 122400 per group for 32 groups
    between two transfers to the int32 total (3.9 M of the 4.19 M its window allows), in both directions."""
    N, K, M, type_ = 256, 32768, 1536, rq.TYPE_W4A4
    blocks = synth.random_weight_blocks(N, K, 5, type_, clip=0.9)
    qs = blocks["qs"].reshape(N, -1)
    qs[0, :] = 0x88888888
    qs[1, :] = 0x77777777
    qs[2, ::2] = 0x88888888
    qs[2, 1::2] = 0x77777777
    blocks["qs"] = qs.reshape(blocks["qs"].shape)
    blocks["sum"] = synth.signed_code_sums(qs).astype(np.int32)[:, None]
    W = rq.W4A4Weight(blocks, type_, DEV)
    x = synth.activations("outlier_channels", M, K, 9)
    x[0, :] = 1.0
    x[1, :] = -1.0
    x[2, :] = np.where((np.arange(K) // 64) % 2 == 0, 1.0, -1.0)
    x[1535, :] = 0.5
    got = run_gpu(W, x)
    sample = [0, 1, 2, 3, 127, 128, 700, 1534, 1535]
    want = oracle.mul_mat(type_, blocks, x[sample], W.clip, n_rot=0)
    assert bits_equal(got[sample], want), first_mismatch(got[sample], want)
    clip = np.float32(0.9)
    unit = np.float32(np.float32(1.0) * clip) / np.float32(3825.0)
    expect = (np.float32(-122400 * 512) * np.float32(16.0)) * unit * blocks["d"][0, 0]
    assert got[0, 0] == np.float32(expect)


@pytest.mark.parametrize("per", [256, 64])
def test_weight_multipliers_extreme_sums(oracle, per):
    """The same extremes on a tensor with weight multipliers (rq.pack_groups, one per block or per 64 inputs): rows of
    all -8 / all +7 codes with multiplier 15 everywhere against q - z = +-15 with m = 255. A group then moves the
    biased accumulator by 15 x 122400 = 1.836 M, so the kernel for such tensors transfers it to the int32 total after
    every second group (3.67 M of the 4.19 M of its window); whole tiles and K slices, both signs."""
    N, K, M, type_ = 300, 4352, 1200, rq.TYPE_W4A4
    rng = np.random.default_rng(17)
    codes = rng.integers(-8, 8, size=(N, K), dtype=np.int8)
    codes[0, :] = -8
    codes[1, :] = 7
    codes[2, :] = np.where((np.arange(K) // 64) % 2 == 0, -8, 7)
    units = np.abs(rng.normal(0.02, 0.005, size=N)).astype(np.float32)
    mults = rng.integers(1, 16, size=(N, K // per), dtype=np.int32)
    mults[0:3, :] = 15
    mults[5, :] = 1
    blocks = rq.pack_groups(codes, units, mults)
    W = rq.W4A4Weight(blocks, type_, DEV)
    x = synth.activations("outlier_channels", M, K, 9)
    x[0, :] = 1.0
    x[1, :] = -1.0
    x[2, :] = np.where((np.arange(K) // 64) % 2 == 0, 1.0, -1.0)
    got = run_gpu(W, x)
    sample = [0, 1, 2, 3, 127, 128, 640, 1199]
    want = oracle.mul_mat(type_, blocks, x[sample], W.clip, n_rot=0)
    assert bits_equal(got[sample], want), first_mismatch(got[sample], want)
    unit = np.float32(1.0) / np.float32(3825.0)
    expect = (np.float32(-15 * 122400 * (K // 64)) * np.float32(16.0)) * unit * units[0]
    assert got[0, 0] == np.float32(expect)


def test_weight_multipliers_at_an_address_the_library_has_not_seen(oracle):
    """The launcher picks the kernel for tensors with weight multipliers from what rq_w4a4_prepare saw. A copy of the
    prepared bytes at another address is unknown to it and takes the other kernel, which must give the same bits."""
    import ctypes
    import torch
    N, K, M, type_ = 520, 2560, 200, rq.TYPE_W4A4H
    blocks, wf = adversarial_weights(oracle, N, K, type_, wgroup=64)
    W = rq.W4A4Weight(blocks, type_, DEV)
    x_np = adversarial_activations(M, K, type_, wf)
    want = oracle.mul_mat(type_, blocks, x_np, W.clip, n_rot=K)
    assert bits_equal(run_gpu(W, x_np), want)
    L = rq.load_library()
    moved = torch.empty(W.prepared.numel() + 4096, dtype=torch.uint8, device=DEV)[2048:2048 + W.prepared.numel()]
    assert moved.data_ptr() % 256 == 0
    moved.copy_(W.prepared)
    x = torch.from_numpy(x_np).to(DEV)
    y = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
    ws = W.workspace(M)
    rc = L.rq_w4a4_mul_mat(type_, moved.data_ptr(), K, N, x.data_ptr(), K, M, y.data_ptr(), N, W.clip, K, ws.data_ptr(),
                           ws.numel(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    got = y.cpu().numpy()
    assert bits_equal(got, want), first_mismatch(got, want)


@pytest.mark.parametrize("M", [65, 128, 129, 300])
def test_token_counts_around_the_tile(oracle, M):
    """One and a few token tiles, partly filled, K = 5120 (every tile cut along K: few tiles, long rows)."""
    N, K, type_ = 520, 5120, rq.TYPE_W4A4H
    blocks, wf = adversarial_weights(oracle, N, K, type_)
    W = rq.W4A4Weight(blocks, type_, DEV)
    x = adversarial_activations(M, K, type_, wf, seed=M)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, blocks, x, W.clip, n_rot=K)
    assert bits_equal(got, want), first_mismatch(got, want)


def test_workspace_without_slabs_runs_every_tile_whole(oracle):
    """A workspace that ends in front of the slabs of the K slices (what the static entry point has for wide batches)
    gives the same bits: the launch then runs every tile whole."""
    N, K, M, type_ = 520, 2560, 200, rq.TYPE_W4A4H
    blocks, wf = adversarial_weights(oracle, N, K, type_)
    W = rq.W4A4Weight(blocks, type_, DEV)
    x_np = adversarial_activations(M, K, type_, wf, seed=3)
    want = oracle.mul_mat(type_, blocks, x_np, W.clip, n_rot=K)
    L = rq.load_library()
    full = L.rq_w4a4_workspace_bytes(type_, K, N, M)
    slabs = 256 * 4 + 256 * 256 * 128 * 4
    assert full > slabs
    x = torch.from_numpy(x_np).to(DEV)
    for nbytes in (full, full - slabs + (1 << 20)):
        ws = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
        y = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
        rc = L.rq_w4a4_mul_mat(type_, W.prepared.data_ptr(), K, N, x.data_ptr(), K, M, y.data_ptr(), N, W.clip, K,
                               ws.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, rc
        torch.cuda.synchronize()
        got = y.cpu().numpy()
        assert bits_equal(got, want), "%d bytes: %s" % (nbytes, first_mismatch(got, want))


def test_int8_gemm_under_rq_gemm_fp6_0():
    env = dict(os.environ)
    env["RQ_GEMM_FP6"] = "0"
    out = subprocess.run([sys.executable, "-u", os.path.join(HERE, "gemm_i8_case.py")], env=env, capture_output=True,
                         text=True, timeout=600)
    assert out.returncode == 0 and "ALL OK" in out.stdout, out.stdout[-3000:] + out.stderr[-2000:]
