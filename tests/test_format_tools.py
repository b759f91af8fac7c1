"""Host-side format tools against what the reference's own tests assert (src/gptq.rs:307-331: byte offsets of
block_w4a4, the two multiplier encodings, nibble extraction, and ggml's dequantizer reading the multipliers the same
way) and against the header semantics of src/convert.rs:99-101 and 876-878. CPU only: no GPU call is made."""
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))

import ruquant_amd as rq  # noqa: E402


def _case(n=64, k=1024, seed=5):
    rng = np.random.default_rng(seed)
    codes = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
    scales = np.abs(rng.normal(0.02, 0.005, size=n)).astype(np.float32)
    return codes, scales


def test_pack_layout_matches_reference_assertions():
    codes, gs = _case()
    n, k = codes.shape
    packed = rq.pack(codes, gs)
    raw = packed.tobytes()
    assert len(raw) == n * (k // 256) * 144
    for o in (0, 17, 63):
        blk = raw[o * (k // 256) * 144 + 144:][:144]          # second block of the row
        assert np.frombuffer(blk[0:4], "<f4")[0] == gs[o]
        assert np.frombuffer(blk[4:8], "<i4")[0] == int(codes[o].astype(np.int64).sum())
        assert np.frombuffer(blk[8:12], "<i4")[0] == k
        assert np.frombuffer(blk[12:16], "<i4")[0] == 0
        for e in (0, 7, 8, 255):
            word = int(np.frombuffer(blk[16 + 4 * (e // 8):20 + 4 * (e // 8)], "<u4")[0])
            nib = (word >> (4 * (e % 8))) & 0xF
            c = nib - 16 if nib >= 8 else nib
            assert c == codes[o, 256 + e]


@pytest.mark.parametrize("per", [1, 4])
def test_pack_groups_encodings_and_dequantizer(per):
    codes, gu = _case(seed=9)
    n, k = codes.shape
    rng = np.random.default_rng(3)
    gm = rng.integers(1, 16, size=(n, per * (k // 256)), dtype=np.uint8)
    gp = rq.pack_groups(codes, gu, gm)
    blk = gp[3, 1]                                            # row 3, block 1
    assert blk["d"] == gu[3]
    if per == 1:
        assert int(blk["sum"]) == (1 << 30 | int(gm[3, 1]))
    else:
        want = 3 << 29
        for g in range(4):
            want |= int(gm[3, 4 + g]) << (4 * g)
        assert int(np.uint32(blk["sum"])) == want
    # the dequantizer reads the multipliers the same way: deq = code * (mult * unit), one rounding per product
    deq = rq.dequantize_rows(gp)
    group = 256 // per
    for i in range(0, n * k, 97):
        o, j = divmod(i, k)
        m = np.float32(gm[o, j // group])
        assert deq[o, j] == np.float32(codes[o, j]) * np.float32(m * gu[o]), i


def test_dequantizer_legacy_header_has_multiplier_one():
    codes, gs = _case(seed=2)
    deq = rq.dequantize_rows(rq.pack(codes, gs))
    assert (deq == codes.astype(np.float32) * gs[:, None]).all()


def test_dequantizer_matches_oracle(oracle):
    codes, gu = _case(n=8, k=512, seed=4)
    gm = np.random.default_rng(1).integers(1, 16, size=(8, 8), dtype=np.uint8)
    blocks = rq.pack_groups(codes, gu, gm)
    want = np.stack([oracle.dequantize_row_w(blocks[r], hadamard=False) for r in range(blocks.shape[0])])
    assert (rq.dequantize_rows(blocks) == want).all()


def test_header_writers():
    codes, gs = _case(n=4, k=512)
    b = rq.pack(codes, gs)
    before = b.copy()
    rq.set_clip(b, 0.85)
    assert (b["pad"][..., 1].view(np.float32) == np.float32(0.85)).all()
    assert rq.resolve_clip(b[0, 0], rq.TYPE_W4A4H) == np.float32(0.85)
    rq.set_clip(b, 0.0)
    assert (b["pad"][..., 1] == 0).all() and rq.resolve_clip(b[0, 0], rq.TYPE_W4A4) == 1.0
    rq.set_rot_len(b, 128)
    assert (b["pad"][..., 0] == 128).all()
    assert rq.tensor_rot(b[0, 0], rq.TYPE_W4A4H, 512) == 128
    # nothing but the two header words changed
    for f in ("d", "sum", "qs"):
        assert (b[f] == before[f]).all()
