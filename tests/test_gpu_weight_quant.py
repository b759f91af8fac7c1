"""GPU parity of the weight-side quantizer and the dequantizers (the types' from_float_ref / to_float, patch lines
2507-2580, 2681-2710, 2738-2773) against the CPU oracle: every byte of every block, every bit of every float."""
import numpy as np
import pytest
import torch

import ruquant_amd as rq
from tests.gpu_util import bits_equal, first_mismatch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
f32 = np.float32


def tensor(N, K, seed):
    """Rows of several characters: gaussian, heavy-tailed, one outlier, group-scaled, flat +-1, all zero."""
    rng = np.random.default_rng(seed)
    w = rng.standard_normal((N, K)).astype(f32) * f32(0.02)
    for r in range(N):
        kind = r % 6
        if kind == 1:
            w[r] = (rng.standard_t(3, size=K) * 0.02).astype(f32)
        elif kind == 2:
            w[r, rng.integers(K)] = 3.0
        elif kind == 3:
            w[r] = (rng.uniform(-1, 1, size=K) * np.exp2((np.arange(K) // 64 + r) % 5 - 2)).astype(f32)
        elif kind == 4:
            w[r] = np.where(rng.uniform(size=K) < 0.5, -1.0, 1.0)
        elif kind == 5 and r % 12 == 5:
            w[r] = 0.0
    return w


def blocks_equal(got, want):
    return got.shape == want.shape and got.tobytes() == want.tobytes()


def block_diff(got, want):
    for name in ("d", "sum", "pad", "qs"):
        bad = np.argwhere(got[name].view(np.uint32) != want[name].view(np.uint32))
        if bad.size:
            i = tuple(bad[0])
            return "%s differs at %s: got %r want %r (%d places)" % (name, i, got[name][i], want[name][i], len(bad))
    return "equal"


@pytest.mark.parametrize("wgroup", [0, 256, 64])
@pytest.mark.parametrize("K", [256, 1536, 5120])
def test_quantize_w4a4_vs_oracle(oracle, K, wgroup):
    N = 37
    w = tensor(N, K, K + wgroup)
    got = rq.quantize_weights(torch.from_numpy(w).to(DEV), rq.TYPE_W4A4, wgroup=wgroup)
    want = oracle.quantize_rows_w(w, wgroup=wgroup)
    assert blocks_equal(got, want), block_diff(got, want)


@pytest.mark.parametrize("K,n_rot,wgroup", [(256, 256, 0), (1536, 1536, 0), (1536, 768, 64), (4096, 4096, 256),
                                             (5120, 5120, 0), (5120, 2560, 0), (5120, 5120, 64), (6144, 6144, 0),
                                             (17408, 17408, 0), (17408, 4352, 256), (11264, 11264, 0)])
def test_quantize_w4a4h_vs_oracle(oracle, K, n_rot, wgroup):
    N = 19
    w = tensor(N, K, K + n_rot + wgroup)
    got = rq.quantize_weights(torch.from_numpy(w).to(DEV), rq.TYPE_W4A4H, n_rot=n_rot, wgroup=wgroup)
    want = oracle.quantize_rows_w(w, hadamard=True, n_rot=n_rot, wgroup=wgroup)
    assert blocks_equal(got, want), block_diff(got, want)


def test_quantize_strided_rows(oracle):
    N, K = 8, 1024
    full = np.zeros((N, K + 64), dtype=f32)
    full[:, :K] = tensor(N, K, 4)
    wd = torch.from_numpy(full).to(DEV)[:, :K]
    got = rq.quantize_weights(wd, rq.TYPE_W4A4H)
    want = oracle.quantize_rows_w(np.ascontiguousarray(full[:, :K]), hadamard=True)
    assert blocks_equal(got, want), block_diff(got, want)


def test_quantize_rejects_bad_arguments():
    w = torch.zeros((4, 512), dtype=torch.float32, device=DEV)
    with pytest.raises(rq.RqError):
        rq.quantize_weights(w, rq.TYPE_W4A4, wgroup=128)
    with pytest.raises(rq.RqError):
        rq.quantize_weights(w, rq.TYPE_W4A4H, n_rot=96)            # no Hadamard of that length
    with pytest.raises(rq.RqError):
        rq.quantize_weights(torch.zeros((4, 384), dtype=torch.float32, device=DEV), rq.TYPE_W4A4)


@pytest.mark.parametrize("K,n_rot,wgroup", [(512, 512, 0), (1536, 1536, 64), (5120, 5120, 256), (5120, 1280, 0),
                                             (17408, 17408, 0), (6144, 6144, 64)])
def test_dequantize_weights_vs_oracle(oracle, K, n_rot, wgroup):
    N = 11
    w = tensor(N, K, 5 * K + wgroup)
    for had, type_ in ((False, rq.TYPE_W4A4), (True, rq.TYPE_W4A4H)):
        blocks = oracle.quantize_rows_w(w, hadamard=had, n_rot=n_rot, wgroup=wgroup)
        got = rq.dequantize(blocks, type_).cpu().numpy()
        want = np.stack([oracle.dequantize_row_w(blocks[r], hadamard=had) for r in range(N)])
        assert bits_equal(got, want), first_mismatch(got, want)


@pytest.mark.parametrize("G", [64, 128, 256])
@pytest.mark.parametrize("K,n_rot", [(512, 512), (5120, 5120), (5120, 2560), (17408, 17408)])
def test_dequantize_activations_vs_oracle(oracle, K, n_rot, G):
    M = 5
    rng = np.random.default_rng(K + G)
    x = (rng.standard_normal((M, K)) * np.exp2(rng.integers(-3, 4, size=(M, K)))).astype(f32)
    for had, type_ in ((False, rq.TYPE_A4), (True, rq.TYPE_A4H)):
        if had:
            blocks = np.stack([oracle.quantize_row_a4h(x[t], 0.9, n_rot, G) for t in range(M)])
        else:
            blocks = np.stack([oracle.quantize_row_a(x[t], 0.9, G) for t in range(M)])
        got = rq.dequantize(blocks, type_).cpu().numpy()
        want = np.stack([oracle.dequantize_row_a(blocks[t], hadamard=had) for t in range(M)])
        assert bits_equal(got, want), first_mismatch(got, want)


def test_quantized_tensor_feeds_the_op(oracle):
    """from_float_ref on the GPU -> the op: same y as the oracle computes from its own quantizer's blocks."""
    N, K, M = 128, 5120, 9
    w = tensor(N, K, 77)
    blocks = rq.quantize_weights(torch.from_numpy(w).to(DEV), rq.TYPE_W4A4H, wgroup=64)
    rq.set_clip(blocks, 0.9)
    x = np.random.default_rng(5).standard_normal((M, K)).astype(f32)
    weight = rq.W4A4Weight(blocks, rq.TYPE_W4A4H, DEV)
    got = rq.mul_mat(weight, torch.from_numpy(x).to(DEV)).cpu().numpy()
    ref_blocks = oracle.quantize_rows_w(w, hadamard=True, wgroup=64)
    rq.set_clip(ref_blocks, 0.9)
    want = oracle.mul_mat(rq.TYPE_W4A4H, ref_blocks, x, f32(0.9), K)
    assert bits_equal(got, want), first_mismatch(got, want)


def test_full_size_tensor_sampled_rows(oracle):
    """A whole 17408 x 5120 tensor (the `down` projection) through the GPU quantizer; the oracle checks a sample of
    rows, and every block of the tensor must carry its row's header."""
    N, K = 5120, 17408
    g = torch.Generator(device=DEV)
    g.manual_seed(1)
    w = torch.randn((N, K), dtype=torch.float32, device=DEV, generator=g) * 0.02
    torch.cuda.synchronize()
    t0 = torch.cuda.Event(enable_timing=True)
    t1 = torch.cuda.Event(enable_timing=True)
    L = rq.load_library()
    ws = torch.empty(L.rq_w4a4_quantize_weights_workspace_bytes(rq.TYPE_W4A4H, K, N, 0), dtype=torch.uint8, device=DEV)
    out = torch.zeros(N * (K // 256) * 144, dtype=torch.uint8, device=DEV)
    import ctypes
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    t0.record()
    rc = L.rq_w4a4_quantize_weights(rq.TYPE_W4A4H, w.data_ptr(), K, N, K, K, 0, out.data_ptr(), ws.data_ptr(),
                                    ws.numel(), st)
    t1.record()
    torch.cuda.synchronize()
    assert rc == 0
    print("quantize 5120 x 17408 W4A4H: %.2f ms" % t0.elapsed_time(t1), flush=True)
    blocks = out.cpu().numpy().view(rq.BLOCK_DTYPE).reshape(N, K // 256)
    assert (blocks["pad"][:, :, 0] == K).all() and (blocks["pad"][:, :, 1] == 0).all()
    assert (blocks["d"] == blocks["d"][:, :1]).all() and (blocks["sum"] == blocks["sum"][:, :1]).all()
    sample = [0, 1, 63, 64, 1000, 2559, 2560, 4095, 5118, 5119]
    wn = w[sample].cpu().numpy()
    want = oracle.quantize_rows_w(wn, hadamard=True)
    assert blocks_equal(blocks[sample], want), block_diff(blocks[sample], want)
