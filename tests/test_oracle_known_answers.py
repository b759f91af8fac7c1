"""Pins the CPU oracle against the known answers printed by the compiled C reference
(tests/golden/reference_known_answers.json) and against closed forms."""
import json
import os

import numpy as np
import pytest

from tests.lcg import act_row, weight_row, fnv64, signed_nibbles

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_known_answers.json")) as f:
    KA = json.load(f)


def bits(x):
    return "%08x" % int(np.asarray(x, dtype=np.float32).view(np.uint32))


@pytest.mark.parametrize("case", KA["hadamard"], ids=lambda c: "k%d" % c["k"])
def test_hadamard_known_answers(oracle, case):
    k = case["k"]
    assert oracle.hadamard_factor(k) == (case["p"], case["m"])
    y = oracle.hadamard(act_row(k))
    assert bits(y[0]) == case["h0"]
    assert bits(y[1]) == case["h1"]
    assert bits(y[-1]) == case["hlast"]
    assert fnv64(y.astype("<f4").tobytes()) == case["fnv64"]


@pytest.mark.parametrize("case", KA["quant"], ids=lambda c: "k%d_%s_%s" % (c["k"], "QH" if c["hadamard"] else "Q", c["clip"]))
def test_quantizer_and_vec_dot_known_answers(oracle, case):
    k = case["k"]
    clip = float(np.float32(float(case["clip"])))
    x = act_row(k)
    a = oracle.quantize_row_a4h(x, clip, k) if case["hadamard"] else oracle.quantize_row_a(x, clip)
    assert bits(a["d"][0]) == case["u"]
    assert "%08x" % (int(a["sum"][0]) & 0xFFFFFFFF) == case["sum0"]
    assert "%08x" % (int(a["pad"][0, 0]) & 0xFFFFFFFF) == case["pad0"]
    assert fnv64(a.tobytes()) == case["fnv64"]
    w = weight_row(k)
    assert int(w["sum"][0]) == KA["row_code_sums"][str(k)]
    assert bits(oracle.vec_dot(w, a)) == case["y"]


def test_zero_row_closed_form(oracle):
    z = KA["zero_row"]
    a = oracle.quantize_row_a(np.zeros(z["k"], dtype=np.float32), z["clip"])
    assert bits(a["d"][0]) == z["u"]
    assert np.float32(2.0) / np.float32(3825.0) == a["d"][0]
    assert all("%08x" % (int(s) & 0xFFFFFFFF) == z["sum0"] for s in a["sum"])
    assert all("%08x" % (int(s) & 0xFFFFFFFF) == z["pad0"] for s in a["pad"][:, 0])
    assert (a["qs"] == int(z["code_word"], 16)).all()


def test_nonnegative_row_has_zero_zero_points(oracle):
    rng = np.random.default_rng(3)
    x = np.maximum(rng.standard_normal(1024).astype(np.float32), 0) ** 2
    a = oracle.quantize_row_a(x, 1.0)
    assert ((a["sum"] & 0xFFFF) == 0).all()
    # widest group gets the full multiplier
    assert ((a["pad"][:, 0].view(np.uint32)[:, None] >> (8 * np.arange(4, dtype=np.uint32))) & 0xFF).max() == 255


@pytest.mark.parametrize("n", [256, 1536, 5120])
def test_hadamard_is_orthogonal_and_transpose_inverts(oracle, n):
    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(np.float32)
    y = oracle.hadamard(x)
    assert abs(float(np.dot(y.astype(np.float64), y.astype(np.float64))) /
               float(np.dot(x.astype(np.float64), x.astype(np.float64))) - 1) < 1e-5
    back = oracle.hadamard(y, transpose=True)
    assert np.abs(back - x).max() < 1e-4


@pytest.mark.parametrize("n", [12 * 4, 20 * 8, 256, 68 * 4])
def test_hadamard_matches_dense_sign_matrix_on_small_integers(oracle, n):
    """On small integers every add is exact, so x H must equal the dense +-1 product times one rounding
    of the scale: pins the Paley matrix orientation and the Sylvester sign pattern."""
    p, m = oracle.hadamard_factor(n)
    A = oracle.paley(p).astype(np.int64) if p > 1 else np.ones((1, 1), dtype=np.int64)
    if p > 1:
        assert (A @ A.T == p * np.eye(p, dtype=np.int64)).all()
    idx = np.arange(m)
    Hm = np.array([[(-1) ** bin(i & j).count("1") for j in idx] for i in idx], dtype=np.int64)
    H = np.kron(A, Hm)  # H[i*m + r, a*m + c] = A[i, a] * Hm[r, c]
    rng = np.random.default_rng(n)
    x = rng.integers(-8, 9, size=n).astype(np.float32)
    want = (x.astype(np.int64) @ H).astype(np.float32) * (np.float32(1.0) / np.sqrt(np.float32(n)))
    got = oracle.hadamard(x)
    assert (got.view(np.uint32) == want.astype(np.float32).view(np.uint32)).all()
    # transposed
    want_t = (x.astype(np.int64) @ H.T).astype(np.float32) * (np.float32(1.0) / np.sqrt(np.float32(n)))
    got_t = oracle.hadamard(x, transpose=True)
    assert (got_t.view(np.uint32) == want_t.view(np.uint32)).all()


def test_factorizations(oracle):
    assert oracle.hadamard_factor(4096) == (1, 4096)
    assert oracle.hadamard_factor(5120) == (20, 256)
    assert oracle.hadamard_factor(6144) == (12, 512)
    assert oracle.hadamard_factor(17408) == (68, 256)
    assert oracle.hadamard_factor(1536) == (12, 128)
    assert oracle.hadamard_factor(1024) == (1, 1024)
    assert oracle.hadamard_factor(4352) == (68, 64)
    assert oracle.hadamard_factor(7 * 256) is None


def brute_vec_dot(w, a):
    """Independent integer restatement from the block layout: per 64-wide group (lsub = 2)."""
    total = 0
    for b in range(w.size):
        cw = signed_nibbles(w["qs"][b]).astype(np.int64)
        ca = signed_nibbles(a["qs"][b]).astype(np.int64)
        lsub = (int(a["sum"][b]) >> 16) & 3
        ngb = 1 << lsub
        per = 256 // ngb
        for sg in range(ngb):
            sl = slice(sg * per, (sg + 1) * per)
            z = (int(a["sum"][b]) >> (4 * sg)) & 0xF
            m = (int(a["pad"][b, 0]) & 0xFFFFFFFF) >> (8 * sg) & 0xFF
            s = int(w["sum"][b]) & 0xFFFFFFFF
            g64 = sg << (2 - lsub)
            kw = (s >> (4 * g64)) & 0xF if (s >> 29) == 3 else (s & 0xF if (s >> 30) == 1 else 1)
            # q - z, summed against the weight codes: acc + (8 - z) colsum
            term = kw * m * int((cw[sl] * (ca[sl] + 8 - z)).sum())
            total += term >> 4  # Python's >> floors, as an arithmetic shift does
    f = np.float32(total)
    return ((f * np.float32(16.0)) * a["d"][0]) * w["d"][0]


@pytest.mark.parametrize("G", [64, 128, 256])
@pytest.mark.parametrize("wsum", ["legacy", "block", "group"])
def test_vec_dot_brute_force(oracle, G, wsum):
    if wsum == "group" and G != 64:
        pytest.skip("weight groups of 64 need activation groups of 64 (reference asserts)")
    rng = np.random.default_rng(G + len(wsum))
    k = 1024
    x = (rng.standard_normal(k) * np.exp2(rng.integers(-3, 4, size=k))).astype(np.float32)
    a = oracle.quantize_row_a(x, 0.9, G)
    w = weight_row(k)
    if wsum == "block":
        w["sum"] = (1 << 30) | rng.integers(1, 16, size=w.size)
    elif wsum == "group":
        ks = rng.integers(1, 16, size=(w.size, 4))
        w["sum"] = ((3 << 29) | ks[:, 0] | ks[:, 1] << 4 | ks[:, 2] << 8 | ks[:, 3] << 12).astype(np.uint32).view(np.int32)
    got = oracle.vec_dot(w, a)
    assert bits(got) == bits(brute_vec_dot(w, a))


def test_clip_precedence(oracle):
    L = oracle.lib()
    assert L.rqo_resolve_clip(-1.0, 0.0) == 1.0
    assert L.rqo_resolve_clip(-1.0, np.float32(0.9)) == np.float32(0.9)
    assert L.rqo_resolve_clip(np.float32(0.85), np.float32(0.9)) == np.float32(0.85)
    assert L.rqo_resolve_clip(0.0, 0.0) == 1.0


def test_mul_mat_equals_rowwise_calls(oracle):
    rng = np.random.default_rng(0)
    K, N, M = 1536, 24, 5
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = oracle.quantize_rows_w(rng.uniform(-1, 1, size=(N, K)).astype(np.float32), hadamard=True)
    y = oracle.mul_mat(oracle.TYPE_W4A4H, w, x, 0.9, n_rot=K, n_threads=3)
    for t in range(M):
        a = oracle.quantize_row_a4h(x[t], 0.9, K)
        for r in range(N):
            assert bits(y[t, r]) == bits(oracle.vec_dot(w[r], a))
