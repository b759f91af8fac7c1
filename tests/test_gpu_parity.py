"""GPU parity: every stage of the HIP path against the CPU oracle, zero tolerance (bit patterns compared)."""
import json
import os

import numpy as np
import pytest
import torch

import ruquant_amd as rq
from ruquant_amd import synth
from tests.gpu_util import bits_equal, first_mismatch, adversarial_weights, adversarial_activations, run_gpu
from tests.lcg import act_row, weight_row, fnv64

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_known_answers.json")) as f:
    KA = json.load(f)

DEV = "cuda:0"


def f32bits(x):
    return "%08x" % int(np.asarray(x, dtype=np.float32).view(np.uint32))


# ---------------------------------------------------------------- Hadamard (kernel 1)

@pytest.mark.parametrize("case", KA["hadamard"], ids=lambda c: "k%d" % c["k"])
def test_hadamard_reference_known_answers(case):
    """The compiled reference's own outputs, no oracle involved."""
    k = case["k"]
    x = torch.from_numpy(act_row(k)[None, :]).to(DEV)
    y = rq.hadamard(x).cpu().numpy()[0]
    assert f32bits(y[0]) == case["h0"] and f32bits(y[1]) == case["h1"] and f32bits(y[-1]) == case["hlast"]
    assert fnv64(y.astype("<f4").tobytes()) == case["fnv64"]


@pytest.mark.parametrize("K,n_rot", [(256, 256), (256, 128), (256, 32), (768, 12), (1536, 1536), (1536, 768),
                                       (4096, 4096), (5120, 5120), (5120, 2560), (6144, 6144), (17408, 17408),
                                       (17408, 4352), (8192, 8192), (32768, 32768), (24576, 24576), (11264, 11264),
                                       (15360, 15360), (18432, 18432), (21504, 21504), (26624, 26624), (27648, 27648),
                                       (20480, 5120), (22528, 22528), (30720, 30720), (21760, 4352), (23040, 4608)])
def test_hadamard_vs_oracle(oracle, K, n_rot):
    rng = np.random.default_rng(K + n_rot)
    M = 3
    x = (rng.standard_normal((M, K)) * np.exp2(rng.integers(-6, 7, size=(M, K)))).astype(np.float32)
    got = rq.hadamard(torch.from_numpy(x).to(DEV), n_rot).cpu().numpy()
    want = np.stack([np.concatenate([oracle.hadamard(x[t, o:o + n_rot]) for o in range(0, K, n_rot)]) for t in range(M)])
    assert bits_equal(got, want), first_mismatch(got, want)


def test_hadamard_signed_zero_and_strided_rows(oracle):
    K = 1536
    x = np.zeros((2, K + 64), dtype=np.float32)
    x[0, :K] = -0.0
    x[1, :K] = np.random.default_rng(0).standard_normal(K).astype(np.float32)
    xd = torch.from_numpy(x).to(DEV)[:, :K]            # row stride K + 64 floats
    got = rq.hadamard(xd).cpu().numpy()
    want = np.stack([oracle.hadamard(x[t, :K]) for t in range(2)])
    assert bits_equal(got, want), first_mismatch(got, want)


# ---------------------------------------------------------------- quantizer (kernel 2)

@pytest.mark.parametrize("case", KA["quant"], ids=lambda c: "k%d_%s_%s" % (c["k"], "QH" if c["hadamard"] else "Q", c["clip"]))
def test_quantizer_reference_known_answers(case):
    k = case["k"]
    clip = float(np.float32(float(case["clip"])))
    x = torch.from_numpy(act_row(k)[None, :]).to(DEV)
    a = rq.quantize_act(x, clip, hadamard_=case["hadamard"])[0]
    assert f32bits(a["d"][0]) == case["u"]
    assert "%08x" % (int(a["sum"][0]) & 0xFFFFFFFF) == case["sum0"]
    assert "%08x" % (int(a["pad"][0, 0]) & 0xFFFFFFFF) == case["pad0"]
    assert fnv64(a.tobytes()) == case["fnv64"]


@pytest.mark.parametrize("K", [256, 1536, 5120, 17408, 32768])
@pytest.mark.parametrize("had", [False, True])
def test_quantizer_blocks_vs_oracle(oracle, K, had):
    rng = np.random.default_rng(K)
    M = 5
    x = (rng.standard_normal((M, K)) * np.exp2((np.arange(K) // 64 % 7 - 3))).astype(np.float32)
    x[1] = 0.0                                   # all-zero token: R = 2
    x[2] = np.abs(x[2])                          # non-negative token: every zero point 0
    x[3, ::2] = 0.0
    clip = float(np.float32(0.9))
    got = rq.quantize_act(torch.from_numpy(x).to(DEV), clip, hadamard_=had)
    for t in range(M):
        want = oracle.quantize_row_a4h(x[t], clip, K) if had else oracle.quantize_row_a(x[t], clip)
        assert got[t].tobytes() == want.tobytes(), "token %d" % t


@pytest.mark.parametrize("K", [18432, 21504, 26624, 27648, 30720])
def test_quantizer_long_rows_with_long_paley_stages(oracle, K):
    """Rows of 72 x 256 (two workgroups still share a compute unit's LDS) and longer ones, where one leaves no room for
    another (the build of the kernel without the register cap): Paley orders 84, 104, 108 and 60 (x 512)."""
    rng = np.random.default_rng(K)
    M = 3
    x = (rng.standard_normal((M, K)) * np.exp2((np.arange(K) // 64 % 5 - 2))).astype(np.float32)
    x[1, 1::3] = 0.0
    clip = float(np.float32(0.85))
    got = rq.quantize_act(torch.from_numpy(x).to(DEV), clip, hadamard_=True)
    for t in range(M):
        want = oracle.quantize_row_a4h(x[t], clip, K)
        assert got[t].tobytes() == want.tobytes(), "token %d" % t


# ---------------------------------------------------------------- MUL_MAT, the reference's test shapes

def _shapes_reference():
    shapes = []
    for m in [1, 3, 8, 17, 64, 200]:
        for k in [256, 512, 1536, 5120, 6144]:
            shapes.append((136, m, k))
    shapes.append((5120, 32, 17408))
    for m in [1, 2, 4, 5, 8, 16, 24, 32, 48, 64, 65, 130]:
        for k in [256, 6144]:
            shapes.append((256, m, k))
    shapes += [(192, 8, 5120), (1024, 8, 5120), (5120, 8, 17408)]
    return shapes


_WCACHE = {}


def _weights(oracle, N, K, type_, wgroup=0):
    key = (N, K, type_, wgroup)
    if key not in _WCACHE:
        blocks, wf = adversarial_weights(oracle, N, K, type_, wgroup=wgroup)
        _WCACHE.clear()            # one at a time: the big ones are tens of MB
        _WCACHE[key] = (blocks, wf, rq.W4A4Weight(blocks, type_, DEV))
    return _WCACHE[key]


@pytest.mark.parametrize("type_", [rq.TYPE_W4A4, rq.TYPE_W4A4H], ids=["w4a4", "w4a4h"])
@pytest.mark.parametrize("N,M,K", sorted(_shapes_reference(), key=lambda s: (s[0], s[2], s[1])),
                         ids=lambda v: str(v))
def test_mul_mat_reference_shapes(oracle, type_, N, M, K):
    blocks, wf, W = _weights(oracle, N, K, type_)
    x = adversarial_activations(M, K, type_, wf)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, blocks, x, W.clip, n_rot=max(W.n_rot, 0))
    assert bits_equal(got, want), first_mismatch(got, want)


@pytest.mark.parametrize("wgroup", [256, 64])
@pytest.mark.parametrize("M", [3, 40])
def test_mul_mat_weight_multipliers(oracle, wgroup, M):
    """Headers that carry integer weight multipliers per block or per 64 inputs (patch lines 40-43)."""
    N, K, type_ = 200, 1536, rq.TYPE_W4A4H
    blocks, wf = adversarial_weights(oracle, N, K, type_, wgroup=wgroup)
    assert ((blocks["sum"].view(np.uint32) >> 30) == 1).all()
    W = rq.W4A4Weight(blocks, type_, DEV)
    x = adversarial_activations(M, K, type_, wf)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, blocks, x, W.clip, n_rot=K)
    assert bits_equal(got, want), first_mismatch(got, want)


@pytest.mark.parametrize("M", [9, 15, 16, 31, 33, 47, 49, 63])
def test_mul_mat_token_counts_between_gemv_and_gemm(oracle, M):
    """Every fill of the 16-token tiles of the kernel that serves 9..64 tokens, with split K and a ragged N."""
    N, K, type_ = 1000, 5120, rq.TYPE_W4A4H
    blocks, wf, W = _weights(oracle, N, K, type_)
    x = adversarial_activations(M, K, type_, wf, seed=M)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, blocks, x, W.clip, n_rot=K)
    assert bits_equal(got, want), first_mismatch(got, want)


@pytest.mark.parametrize("type_", [rq.TYPE_W4A4, rq.TYPE_W4A4H], ids=["w4a4", "w4a4h"])
@pytest.mark.parametrize("M", [1, 7, 70])
def test_mul_mat_longest_row(oracle, type_, M):
    """K = 32768, the longest row the op takes (RQ_MAX_K): one Sylvester transform of 2^15, 512 groups, all three
    product kernels."""
    N, K = 128, 32768
    blocks, wf, W = _weights(oracle, N, K, type_)
    x = adversarial_activations(M, K, type_, wf, seed=3 * M)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, blocks, x, W.clip, n_rot=max(W.n_rot, 0))
    assert bits_equal(got, want), first_mismatch(got, want)


@pytest.mark.parametrize("M", [2, 70])
def test_mul_mat_long_row_long_paley_stage(oracle, M):
    """K = 84 x 256: the activation kernel that has a compute unit to itself, feeding the GEMV and the GEMM."""
    N, K, type_ = 136, 21504, rq.TYPE_W4A4H
    blocks, wf, W = _weights(oracle, N, K, type_)
    x = adversarial_activations(M, K, type_, wf, seed=5 * M)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, blocks, x, W.clip, n_rot=max(W.n_rot, 0))
    assert bits_equal(got, want), first_mismatch(got, want)


@pytest.mark.parametrize("N,K,M,wgroup,type_", [(6144, 1024, 512, 0, rq.TYPE_W4A4H), (6100, 1536, 500, 0, rq.TYPE_W4A4H),
                                                (6144, 1024, 450, 256, rq.TYPE_W4A4), (6144, 768, 512, 64, rq.TYPE_W4A4H)])
def test_gemm_half_tiles(oracle, N, K, M, wgroup, type_):
    """Shapes whose wide tiles would not fill one round of the chip and whose narrow tiles need two: the launch plan
    runs them as half tiles (256 rows x 64 tokens; 24 row tiles x 8 token tiles = 192 workgroups). Whole and ragged
    token and row counts, with and without weight multipliers."""
    blocks, wf = adversarial_weights(oracle, N, K, type_, wgroup=wgroup)
    W = rq.W4A4Weight(blocks, type_, DEV)
    x = adversarial_activations(M, K, type_, wf, seed=M)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, blocks, x, W.clip, n_rot=max(W.n_rot, 0))
    assert bits_equal(got, want), first_mismatch(got, want)


def test_gemm_wide_tiles_longest_row_extreme_sums(oracle):
    """K = 32768 on the wide tiles of the MFMA GEMM with inputs that drive the integer sums to their ends: rows whose
    codes are all -8 or all +7 against tokens that quantize to q - z = +15 or -15 with m = 255 in every one of the
    512 groups (a token of equal positive values: lo = 0, z = 0, every q clamps to 15; of equal negative values:
    z = 15, q = 0). The low-digit accumulator then carries 512 floors of magnitude 480 above its low byte, the
    high-digit accumulator 512 x 491520. 16 row tiles x 12 token tiles = 192 tiles: the launch plan runs them wide
    (one round of wide tiles is cheaper than three rounds of narrow ones). Checked on a sample of tokens (tokens are
    independent: the oracle gets the sampled rows of x)."""
    N, K, M, type_ = 4096, 32768, 1536, rq.TYPE_W4A4
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
    x[3, :] = np.where(np.arange(K) % 2 == 0, 3.0, -3.0)
    x[1535, :] = 0.5
    got = run_gpu(W, x)
    sample = [0, 1, 2, 3, 4, 127, 128, 700, 1534, 1535]
    want = oracle.mul_mat(type_, blocks, x[sample], W.clip, n_rot=0)
    assert bits_equal(got[sample], want), first_mismatch(got[sample], want)
    # closed form of the first extreme, independent of the oracle: every group contributes floor(255 x (-8 x 15 x 64)
    # / 16) = -122400, the token's unit is (1.0 x clip) / 3825
    clip = np.float32(0.9)
    unit = np.float32(np.float32(1.0) * clip) / np.float32(3825.0)
    expect = (np.float32(-122400 * 512) * np.float32(16.0)) * unit * blocks["d"][0, 0]
    assert got[0, 0] == np.float32(expect)


def test_mul_mat_block_diagonal_rotation(oracle):
    """Hadamard length shorter than the row (pad[0] = K / 4), as ruquant convert --rot-blocks writes."""
    N, K, M, type_ = 128, 6144, 9, rq.TYPE_W4A4H
    blocks, wf = adversarial_weights(oracle, N, K, type_, n_rot=K // 4)
    W = rq.W4A4Weight(blocks, type_, DEV)
    assert W.n_rot == K // 4
    x = adversarial_activations(M, K, type_, wf)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, blocks, x, W.clip, n_rot=K // 4)
    assert bits_equal(got, want), first_mismatch(got, want)


def test_converter_tools_feed_the_op(oracle):
    """Blocks built by the format tools (pack_groups, set_clip, set_rot_len), as the reference's converter writes a
    tensor, run through the op: header clip and rotation length are what the kernels use."""
    N, K, M, type_ = 192, 2048, 5, rq.TYPE_W4A4H
    rng = np.random.default_rng(11)
    codes = rng.integers(-8, 8, size=(N, K), dtype=np.int8)
    units = np.abs(rng.normal(0.02, 0.005, size=N)).astype(np.float32)
    mults = rng.integers(1, 16, size=(N, K // 64), dtype=np.uint8)
    blocks = rq.pack_groups(codes, units, mults)
    rq.set_clip(blocks, 0.8)
    rq.set_rot_len(blocks, 512)
    W = rq.W4A4Weight(blocks, type_, DEV)
    assert W.clip == np.float32(0.8) and W.n_rot == 512
    x = synth.activations("student_t4", M, K, 7)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, blocks, x, np.float32(0.8), n_rot=512)
    assert bits_equal(got, want), first_mismatch(got, want)


def test_mul_mat_strided_input_and_output(oracle):
    N, K, M, type_ = 320, 1536, 6, rq.TYPE_W4A4
    blocks, wf = adversarial_weights(oracle, N, K, type_)
    W = rq.W4A4Weight(blocks, type_, DEV)
    x = adversarial_activations(M, K, type_, wf)
    xd = torch.zeros((M, K + 128), dtype=torch.float32, device=DEV)
    xd[:, :K] = torch.from_numpy(x).to(DEV)
    out = torch.full((M, N + 32), -7.0, dtype=torch.float32, device=DEV)
    rq.mul_mat(W, xd[:, :K], out=out[:, :N])
    torch.cuda.synchronize()
    want = oracle.mul_mat(type_, blocks, x, W.clip)
    got = out.cpu().numpy()
    assert bits_equal(got[:, :N], want), first_mismatch(got[:, :N], want)
    assert (got[:, N:] == -7.0).all()


def test_fused_matches_separate(oracle):
    K, M, type_ = 5120, 4, rq.TYPE_W4A4H
    ws, bl = [], []
    for i, N in enumerate([384, 64, 1024]):
        b = synth.random_weight_blocks(N, K, 10 + i, type_, clip=0.9)
        bl.append(b)
        ws.append(rq.W4A4Weight(b, type_, DEV))
    x = synth.activations("outlier_channels", M, K, 5)
    xd = torch.from_numpy(x).to(DEV)
    outs = rq.mul_mat_fused(ws, xd)
    torch.cuda.synchronize()
    for b, w, o in zip(bl, ws, outs):
        want = oracle.mul_mat(type_, b, x, w.clip, n_rot=K)
        assert bits_equal(o.cpu().numpy(), want), first_mismatch(o.cpu().numpy(), want)


@pytest.mark.parametrize("one_launch", [True, False], ids=["one_launch", "launch_per_weight"])
@pytest.mark.parametrize("M", [1, 3, 5, 8, 16, 23, 40, 64, 130])
def test_fused_launch_forms(oracle, M, one_launch):
    """Three weights in one call: legacy headers, weight multipliers (so the per-weight flag word matters) and a row
    count that is not a multiple of the panel; with split-K cells for all rows (one launch of the streaming kernels)
    and with cells for the largest weight only (a launch per weight)."""
    K, type_ = 1536, rq.TYPE_W4A4H
    rng = np.random.default_rng(M)
    ws, bl = [], []
    for i, N in enumerate([384, 96, 1024]):
        if i == 1:
            codes = rng.integers(-8, 8, size=(N, K), dtype=np.int8)
            units = np.abs(rng.normal(0.02, 0.005, size=N)).astype(np.float32)
            mults = rng.integers(1, 16, size=(N, K // 64), dtype=np.uint8)
            b = rq.pack_groups(codes, units, mults)
            rq.set_rot_len(b, K)
            rq.set_clip(b, 0.9)
        else:
            b = synth.random_weight_blocks(N, K, 20 + i, type_, clip=0.9)
        bl.append(b)
        ws.append(rq.W4A4Weight(b, type_, DEV))
    x = synth.activations("student_t4", M, K, 7 + M)
    xd = torch.from_numpy(x).to(DEV)
    L = rq.load_library()
    nbytes = rq.fused_workspace_bytes(ws, M) if one_launch else L.rq_w4a4_workspace_bytes(type_, K, 1024, M)
    work = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    for rep in range(2):                       # the second call meets the cells the first one left
        outs = rq.mul_mat_fused(ws, xd, workspace=work)
        torch.cuda.synchronize()
        for b, w, o in zip(bl, ws, outs):
            want = oracle.mul_mat(type_, b, x, w.clip, n_rot=K)
            assert bits_equal(o.cpu().numpy(), want), first_mismatch(o.cpu().numpy(), want)


# ---------------------------------------------------------------- the five benchmark configurations

def test_config1_w4a4_k4096_n1024_m1(oracle):
    K, N, M = 4096, 1024, 1
    blocks = synth.random_weight_blocks(N, K, 0, rq.TYPE_W4A4)
    W = rq.W4A4Weight(blocks, rq.TYPE_W4A4, DEV)
    assert W.clip == 1.0
    x = synth.activations("normal", M, K, 0)
    got = run_gpu(W, x)
    want = oracle.mul_mat(rq.TYPE_W4A4, blocks, x, 1.0)
    assert bits_equal(got, want), first_mismatch(got, want)


@pytest.mark.parametrize("M", [1, 2, 4, 8])
def test_config2_decode_gemv(oracle, M):
    K, N = 5120, 5120
    blocks = synth.random_weight_blocks(N, K, 2, rq.TYPE_W4A4H, clip=0.9)
    W = rq.W4A4Weight(blocks, rq.TYPE_W4A4H, DEV)
    assert W.clip == float(np.float32(0.9)) and W.n_rot == K
    x = synth.activations("outlier_channels", M, K, 2)
    got = run_gpu(W, x)
    want = oracle.mul_mat(rq.TYPE_W4A4H, blocks, x, W.clip, n_rot=K)
    assert bits_equal(got, want), first_mismatch(got, want)


@pytest.mark.parametrize("M", [64, 512, 2048])
def test_config3_prefill_gemm(oracle, M):
    K, N = 5120, 17408
    blocks = synth.random_weight_blocks(N, K, 3, rq.TYPE_W4A4H)
    W = rq.W4A4Weight(blocks, rq.TYPE_W4A4H, DEV)
    clip = float(np.float32(0.85))                # RQ_ACT_CLIP_H=0.85 in the reference's run; passed explicitly
    x = synth.activations("student_t4", M, K, 3)
    y = rq.mul_mat(W, torch.from_numpy(x).to(DEV), clip=clip)
    torch.cuda.synchronize()
    got = y.cpu().numpy()
    want = oracle.mul_mat(rq.TYPE_W4A4H, blocks, x, clip, n_rot=K)
    assert bits_equal(got, want), first_mismatch(got, want)


@pytest.mark.parametrize("type_,K,N,n_rot,mult", [
    (rq.TYPE_W4A4H, 5120, 17408, 5120, 0),     # the headline: one whole panel per workgroup and a quad of the remainder
    (rq.TYPE_W4A4H, 5120, 17408, 5120, 256),   # ... with a weight multiplier per block
    (rq.TYPE_W4A4H, 5120, 17408, 5120, 64),    # ... per group of 64
    (rq.TYPE_W4A4H, 5120, 16384, 5120, 0),     # whole panels only
    (rq.TYPE_W4A4H, 5120, 33216, 5120, 0),     # two whole panels per workgroup, 7 remainder panels
    (rq.TYPE_W4A4H, 6144, 16576, 6144, 0),     # 12 groups per stream wavefront with remainder items (H12 x H512)
    (rq.TYPE_W4A4H, 6144, 16576, 6144, 64),
    (rq.TYPE_W4A4H, 6144, 16384, 6144, 0),     # 12 groups, no remainder
    (rq.TYPE_W4A4H, 10240, 16448, 10240, 0),   # two rounds of 10 groups per panel (H20 x H512)
    (rq.TYPE_W4A4H, 12288, 16448, 12288, 256), # two rounds of 12 groups (H12 x H1024)
    (rq.TYPE_W4A4H, 8192, 16640, 8192, 0),     # 16 groups per wavefront: 12 + 4 and clamped loads, no Paley stage
    (rq.TYPE_W4A4H, 16384, 16448, 16384, 0),   # the longest row the kernel takes: 32 groups per wavefront, three rounds
    (rq.TYPE_W4A4H, 5120, 16448, 2560, 0),     # block-diagonal rotation (H20 x H128 twice)
    (rq.TYPE_W4A4, 4096, 16448, 0, 0),         # no rotation: 8 groups per wavefront in a round of 10
    (rq.TYPE_W4A4, 6144, 17408, 0, 64),
])
def test_one_token_whole_panels(oracle, type_, K, N, n_rot, mult):
    """One token against weights of at least 256 panels of 64 rows, where every workgroup of the one-launch kernel
    streams whole panels (its stream wavefronts hold 10 or 12 groups per round, the first ones requested before
    anything else) beside its share of the remainder. `mult`: integer weight multipliers in the block headers, one
    per block of 256 codes or one per group of 64 (reference patch lines 38-43)."""
    had = type_ == rq.TYPE_W4A4H
    blocks = synth.random_weight_blocks(N, K, 11, type_, clip=0.9, n_rot=n_rot if had else None)
    rng = np.random.default_rng(13)
    if mult == 256:
        blocks["sum"] = ((1 << 30) | rng.integers(1, 16, size=blocks["sum"].shape)).astype(np.int32)
    elif mult == 64:
        k = rng.integers(1, 16, size=blocks["sum"].shape + (4,))
        blocks["sum"] = ((3 << 29) | k[..., 0] | (k[..., 1] << 4) | (k[..., 2] << 8) | (k[..., 3] << 12)).astype(np.int32)
    W = rq.W4A4Weight(blocks, type_, DEV)
    x = synth.activations("outlier_channels", 1, K, 12)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, blocks, x, W.clip, n_rot=n_rot if had else 0)
    assert bits_equal(got, want), first_mismatch(got, want)


@pytest.mark.parametrize("type_,K,N,mult", [
    (rq.TYPE_W4A4H, 5120, 10240, 0),     # 160 panels: the fewest that run as one whole panel per workgroup (K >= 5120)
    (rq.TYPE_W4A4H, 5120, 16320, 64),    # 255 panels, weight multipliers per group
    (rq.TYPE_W4A4H, 5120, 12000, 0),     # 187.5 panels: the last one is ragged
    (rq.TYPE_W4A4H, 6144, 10304, 256),   # 161 panels of 12 groups per wavefront
    (rq.TYPE_W4A4, 4096, 14400, 0),      # 225 panels of a shorter row (from 7/8 of the compute units on)
    (rq.TYPE_W4A4H, 5120, 9216, 0),      # 144 panels: still dealt in quads, 14 items per wavefront in flight
    (rq.TYPE_W4A4H, 5120, 7168, 0),      # 7 quads per workgroup (runs start inside octets)
    (rq.TYPE_W4A4, 4096, 13056, 64),     # 204 panels of a shorter row, dealt in quads: 16 items in flight
    (rq.TYPE_W4A4H, 10240, 4992, 0),     # long rows, few of them: 40 blocks per octet, 20 items in flight
    (rq.TYPE_W4A4H, 16384, 4160, 0),     # two rounds of 26 items
])
def test_one_token_between_one_and_two_rounds_of_panels(oracle, type_, K, N, mult):
    """One token against weights of fewer panels than compute units. From 5/8 of them on (7/8 for rows shorter than
    5120) every workgroup takes one whole panel and the other compute units stay idle; below, the rows are dealt in
    quads over all compute units, a wavefront's items all in flight in the smallest of the forms for 12, 14, ... 26
    items that holds them."""
    had = type_ == rq.TYPE_W4A4H
    blocks = synth.random_weight_blocks(N, K, 31, type_, clip=0.9, n_rot=K if had else None)
    rng = np.random.default_rng(17)
    if mult == 256:
        blocks["sum"] = ((1 << 30) | rng.integers(1, 16, size=blocks["sum"].shape)).astype(np.int32)
    elif mult == 64:
        k = rng.integers(1, 16, size=blocks["sum"].shape + (4,))
        blocks["sum"] = ((3 << 29) | k[..., 0] | (k[..., 1] << 4) | (k[..., 2] << 8) | (k[..., 3] << 12)).astype(np.int32)
    W = rq.W4A4Weight(blocks, type_, DEV)
    x = synth.activations("outlier_channels", 1, K, 19)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, blocks, x, W.clip, n_rot=K if had else 0)
    assert bits_equal(got, want), first_mismatch(got, want)


def test_one_token_fused_weights_as_whole_panels_on_fewer_workgroups(oracle):
    """Three weights in one call whose panels together (96 + 16 + 56 = 168, the last one ragged) run as one whole panel
    per workgroup: a workgroup finds its weight from the panel index."""
    K, type_ = 5120, rq.TYPE_W4A4H
    ws, bl = [], []
    for i, N in enumerate([6144, 1024, 3560]):
        b = synth.random_weight_blocks(N, K, 40 + i, type_, clip=0.9)
        bl.append(b)
        ws.append(rq.W4A4Weight(b, type_, DEV))
    x = synth.activations("student_t4", 1, K, 23)
    xd = torch.from_numpy(x).to(DEV)
    outs = rq.mul_mat_fused(ws, xd)
    torch.cuda.synchronize()
    for b, w, o in zip(bl, ws, outs):
        want = oracle.mul_mat(type_, b, x, w.clip, n_rot=K)
        assert bits_equal(o.cpu().numpy(), want), first_mismatch(o.cpu().numpy(), want)


@pytest.mark.parametrize("K,n_rot", [(5120, 5120), (6144, 6144), (10240, 10240), (3072, 3072), (5120, 2560), (12288, 12288)])
@pytest.mark.parametrize("row", ["zeros", "one_spike", "constant", "negative_constant", "signed_zeros", "alternating",
                                 "one_group_only", "tiny"])
def test_one_token_rows_that_press_the_group_ranges(oracle, K, n_rot, row):
    """One token whose rotated row has groups without a negative value, without a positive one, all zero, or a range
    far below the token's widest: the one-launch kernel reduces a group's range over the lanes of the register that
    holds the group (bit patterns compared as integers, an identity for absent registers) and must land on the
    reference's min / max chain from 0 (reference patch lines 2646-2654) in every such case. A constant row rotates
    into a single non-zero value per Sylvester chunk; a spike rotates into a row of equal magnitudes."""
    N, type_ = 192, rq.TYPE_W4A4H
    blocks = synth.random_weight_blocks(N, K, 21, type_, clip=1.0, n_rot=n_rot)
    W = rq.W4A4Weight(blocks, type_, DEV)
    x = np.zeros((1, K), np.float32)
    if row == "one_spike":
        x[0, 77] = 3.0
    elif row == "constant":
        x[0, :] = 0.25
    elif row == "negative_constant":
        x[0, :] = -1.5
    elif row == "signed_zeros":
        x[0, ::2] = -0.0
        x[0, 5] = 1.0
        x[0, 6] = -1.0
    elif row == "alternating":
        x[0, :] = np.where(np.arange(K) % 2 == 0, 1.0, -1.0)
    elif row == "one_group_only":
        x[0, :] = synth.activations("outlier_channels", 1, K, 5)[0] * (np.arange(K) // 64 == 3)
    elif row == "tiny":
        x[0, :] = synth.activations("outlier_channels", 1, K, 6)[0] * np.float32(1e-30)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, blocks, x, W.clip, n_rot=n_rot)
    assert bits_equal(got, want), first_mismatch(got, want)


@pytest.mark.parametrize("M", [1, 12, 13, 16, 2048])   # (12 / 13: the rotation goes from items of two outputs to four)
def test_config4_down_projection(oracle, M):
    K, N = 17408, 5120
    blocks = synth.random_weight_blocks(N, K, 4, rq.TYPE_W4A4H)
    W = rq.W4A4Weight(blocks, rq.TYPE_W4A4H, DEV)
    x = synth.activations("relu2", M, K, 4)
    got = run_gpu(W, x)
    want = oracle.mul_mat(rq.TYPE_W4A4H, blocks, x, 1.0, n_rot=K)
    assert bits_equal(got, want), first_mismatch(got, want)


@pytest.mark.parametrize("M", [16, 1, 5, 40])
def test_config5_transformer_layer_chain(oracle, M):
    """Seven matmuls chained along the layer's dataflow: q, k, v <- x0; o <- q; gate, up <- o; down <- up. M = 16 is the
    benchmark configuration; 1 and 5 take the GEMV (fused calls in one launch), 40 the two-token-block skinny kernel."""
    type_ = rq.TYPE_W4A4H
    shapes = dict(q=(5120, 6144), k=(5120, 1024), v=(5120, 1024), o=(6144, 5120), gate=(5120, 17408),
                  up=(5120, 17408), down=(17408, 5120))
    blocks = {n: synth.random_weight_blocks(No, Ki, 100 + i, type_) for i, (n, (Ki, No)) in enumerate(shapes.items())}
    W = {n: rq.W4A4Weight(b, type_, DEV) for n, b in blocks.items()}
    x0 = synth.activations("normal", M, 5120, 1)
    xd = torch.from_numpy(x0).to(DEV)
    q, k, v = rq.mul_mat_fused([W["q"], W["k"], W["v"]], xd)
    o = rq.mul_mat(W["o"], q)
    gate, up = rq.mul_mat_fused([W["gate"], W["up"]], o)
    down = rq.mul_mat(W["down"], up)
    torch.cuda.synchronize()
    ref = lambda n, x: oracle.mul_mat(type_, blocks[n], x, 1.0, n_rot=shapes[n][0])
    rq_, rk, rv = ref("q", x0), ref("k", x0), ref("v", x0)
    ro = ref("o", rq_)
    rg, ru = ref("gate", ro), ref("up", ro)
    rd = ref("down", ru)
    for name, got, want in [("q", q, rq_), ("k", k, rk), ("v", v, rv), ("o", o, ro), ("gate", gate, rg),
                            ("up", up, ru), ("down", down, rd)]:
        g = got.cpu().numpy()
        assert bits_equal(g, want), name + ": " + first_mismatch(g, want)


@pytest.mark.parametrize("wgroup", [0, 64], ids=["legacy", "wgroup64"])
@pytest.mark.parametrize("N,M", [(8300, 1024), (16500, 520)])
def test_gemm_leftover_rows(oracle, N, M, wgroup):
    """More than 256 wide tiles with a few rows left over: whole wide rounds plus a tail that runs through the skinny
    kernel (a sub-range of the panels, blocks of 32 tokens, the last panel partly filled)."""
    K, type_ = 256, rq.TYPE_W4A4H
    blocks, wf, W = _weights(oracle, N, K, type_, wgroup=wgroup)
    x = adversarial_activations(M, K, type_, wf, seed=N + M)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, blocks, x, W.clip, n_rot=K)
    assert bits_equal(got, want), first_mismatch(got, want)


@pytest.mark.parametrize("type_", [rq.TYPE_W4A4, rq.TYPE_W4A4H], ids=["w4a4", "w4a4h"])
@pytest.mark.parametrize("M", [33, 50, 64])
def test_skinny_all_tokens_in_one_workgroup_with_multipliers(oracle, M, type_):
    """Long rows (K = 10240) at 33..64 tokens: the skinny kernel takes all tokens in one workgroup (four token tiles
    per wavefront, single-plane activations); here with weight multipliers per 64 inputs and a partly filled panel."""
    N, K = 200, 10240
    rng = np.random.default_rng(M)
    codes = rng.integers(-8, 8, size=(N, K), dtype=np.int8)
    units = np.abs(rng.normal(0.02, 0.005, size=N)).astype(np.float32)
    mults = rng.integers(1, 16, size=(N, K // 64), dtype=np.uint8)
    b = rq.pack_groups(codes, units, mults)
    rq.set_clip(b, 0.9)
    W = rq.W4A4Weight(b, type_, DEV)
    x = synth.activations("student_t4", M, K, 3 + M)
    got = run_gpu(W, x)
    want = oracle.mul_mat(type_, b, x, W.clip, n_rot=K)
    assert bits_equal(got, want), first_mismatch(got, want)


# ---------------------------------------------------------------- properties that hold at any size

@pytest.mark.parametrize("M", [1, 8, 16, 200])
def test_hip_graph_replays_match_eager(oracle, M):
    """The steady-state call is graph safe (no allocation, no synchronization, no memset nodes): capture it once,
    replay it with fresh inputs and eager work in between, and every replay must equal the oracle."""
    N, K, type_ = 320, 1536, rq.TYPE_W4A4H
    blocks, wf, W = _weights(oracle, N, K, type_)
    x = torch.zeros((M, K), dtype=torch.float32, device=DEV)
    y = torch.zeros((M, N), dtype=torch.float32, device=DEV)
    ws = W.workspace(M)
    xs = [adversarial_activations(M, K, type_, wf, seed=100 + i) for i in range(3)]
    x.copy_(torch.from_numpy(xs[0]))
    rq.mul_mat(W, x, out=y, workspace=ws)          # warm-up outside capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        rq.mul_mat(W, x, out=y, workspace=ws)
    for i in range(3):
        x.copy_(torch.from_numpy(xs[i]))
        y.fill_(-1.0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        want = oracle.mul_mat(type_, blocks, xs[i], W.clip, n_rot=K)
        got = y.cpu().numpy()
        assert bits_equal(got, want), "replay %d: %s" % (i, first_mismatch(got, want))


def test_rows_are_independent_and_calls_repeatable(oracle):
    """A token's output must not depend on its neighbours or on the path taken (GEMV at M=1 vs GEMM inside M=300);
    a second call with the same workspace must reproduce the first (split-K scratch left clean)."""
    K, N, type_ = 5120, 1088, rq.TYPE_W4A4H
    blocks = synth.random_weight_blocks(N, K, 7, type_, clip=0.9)
    W = rq.W4A4Weight(blocks, type_, DEV)
    x = synth.activations("student_t4", 300, K, 8)
    xd = torch.from_numpy(x).to(DEV)
    ws = W.workspace(300)
    big = rq.mul_mat(W, xd, workspace=ws).clone()
    again = rq.mul_mat(W, xd, workspace=ws).clone()
    assert torch.equal(big, again)
    for t in [0, 7, 131, 299]:
        one = rq.mul_mat(W, xd[t:t + 1], workspace=ws)
        assert torch.equal(one[0], big[t]), t
    five = rq.mul_mat(W, xd[10:15], workspace=ws)
    assert torch.equal(five, big[10:15])
