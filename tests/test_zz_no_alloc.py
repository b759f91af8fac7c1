"""rq_w4a4_mul_mat_static (the entry point that allocates nothing: its workspace is an array inside the library's code
object) against rq_w4a4_mul_mat with a caller-owned workspace, through the C ABI, bit for bit. Every pair of calls
shares the one static array, and the second call of a pair is the smaller problem: what the first left in the array
must not leak into it."""
import ctypes

import numpy as np
import pytest
import torch

import ruquant_amd as rq
from ruquant_amd import synth
from tests.gpu_util import bits_equal, first_mismatch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
RQ_E_LIMIT = -4


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _both(L, W, x_np, clip):
    """(y through rq_w4a4_mul_mat_static, y through rq_w4a4_mul_mat) for one problem."""
    M, K = x_np.shape
    x = torch.from_numpy(x_np).to(DEV)
    n_rot = max(W.n_rot, 0)
    y_static = torch.full((M, W.N), float("nan"), dtype=torch.float32, device=DEV)
    rc = L.rq_w4a4_mul_mat_static(W.type, W.prepared.data_ptr(), K, W.N, x.data_ptr(), K, M, y_static.data_ptr(), W.N,
                                  clip, n_rot, _stream())
    assert rc == 0, rc
    ws = W.workspace(M)
    y_ws = torch.full((M, W.N), float("nan"), dtype=torch.float32, device=DEV)
    rc = L.rq_w4a4_mul_mat(W.type, W.prepared.data_ptr(), K, W.N, x.data_ptr(), K, M, y_ws.data_ptr(), W.N, clip,
                           n_rot, ws.data_ptr(), ws.numel(), _stream())
    assert rc == 0, rc
    torch.cuda.synchronize()
    return y_static.cpu().numpy(), y_ws.cpu().numpy()


# (type, K, N, M) of the first call, then of the second, smaller one; the pairs cross the three product paths
PAIRS = [
    ((rq.TYPE_W4A4H, 5120, 1088, 3), (rq.TYPE_W4A4H, 1536, 192, 1)),        # GEMV, then a smaller GEMV
    ((rq.TYPE_W4A4H, 5120, 1024, 48), (rq.TYPE_W4A4H, 5120, 1024, 5)),      # skinny MFMA kernel, fewer tokens
    ((rq.TYPE_W4A4H, 6144, 512, 200), (rq.TYPE_W4A4, 512, 136, 17)),        # tiled GEMM, then skinny on another type
    ((rq.TYPE_W4A4H, 17408, 320, 16), (rq.TYPE_W4A4H, 17408, 320, 2)),      # two-step activation side, then GEMV
    ((rq.TYPE_W4A4, 4096, 1024, 130), (rq.TYPE_W4A4, 4096, 1024, 3)),       # GEMM leaves its planes where the GEMV's cells go
    ((rq.TYPE_W4A4H, 2560, 2048, 300), (rq.TYPE_W4A4H, 2560, 2048, 9)),     # the same in front of the skinny kernel's cells
]


@pytest.mark.parametrize("first,second", PAIRS, ids=lambda p: "%d_k%d_n%d_m%d" % p)
def test_static_workspace_matches_caller_workspace(oracle, first, second):
    L = rq.load_library()
    for i, (type_, K, N, M) in enumerate((first, second)):
        blocks = synth.random_weight_blocks(N, K, 10 + i, type_, clip=0.9 if i == 0 else 0.0)
        W = rq.W4A4Weight(blocks, type_, DEV)
        x_np = synth.activations("outlier_channels" if i == 0 else "student_t4", M, K, 20 + i)
        got, want = _both(L, W, x_np, W.clip)
        assert bits_equal(got, want), "call %d: %s" % (i + 1, first_mismatch(got, want))
        if i == 1:
            ref = oracle.mul_mat(type_, blocks, x_np, W.clip, n_rot=max(W.n_rot, 0))
            assert bits_equal(got, ref), "call 2 vs the CPU oracle: %s" % first_mismatch(got, ref)


def test_static_call_allocates_nothing_and_can_be_captured(oracle):
    """Free device memory is the same before and after eager calls, and a HIP graph that holds static calls of the three
    small-batch paths (1, 3 and 16 tokens; capture forbids allocation) replays to the oracle's bits every time."""
    L = rq.load_library()
    type_, K, N = rq.TYPE_W4A4H, 5120, 1088
    blocks = synth.random_weight_blocks(N, K, 31, type_, clip=0.9)
    W = rq.W4A4Weight(blocks, type_, DEV)
    probs = []
    for M in (1, 3, 16):
        x_np = synth.activations("outlier_channels", M, K, 40 + M)
        probs.append((M, x_np, torch.from_numpy(x_np).to(DEV), torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)))

    def run_all():
        for M, _, x, y in probs:
            rc = L.rq_w4a4_mul_mat_static(type_, W.prepared.data_ptr(), K, N, x.data_ptr(), K, M, y.data_ptr(), N, W.clip,
                                          K, _stream())
            assert rc == 0, rc

    run_all()
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        run_all()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    want = [oracle.mul_mat(type_, blocks, x_np, W.clip, n_rot=K) for _, x_np, _, _ in probs]
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        run_all()
    for replay in range(3):
        for _, _, _, y in probs:
            y.fill_(float("nan"))          # eager work between the replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for (M, _, _, y), ref in zip(probs, want):
            got = y.cpu().numpy()
            assert bits_equal(got, ref), "replay %d, M=%d: %s" % (replay, M, first_mismatch(got, ref))


def test_static_workspace_refuses_what_does_not_fit():
    L = rq.load_library()
    K, N, M = 32768, 17408, 16
    assert L.rq_w4a4_workspace_bytes(rq.TYPE_W4A4H, K, N, M) > (16 << 20)
    dummy = torch.zeros(1024, dtype=torch.float32, device=DEV)
    rc = L.rq_w4a4_mul_mat_static(rq.TYPE_W4A4H, dummy.data_ptr(), K, N, dummy.data_ptr(), K, M, dummy.data_ptr(), N,
                                  1.0, K, _stream())
    assert rc == RQ_E_LIMIT
    torch.cuda.synchronize()
