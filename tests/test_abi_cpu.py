"""CPU-side checks of the shipped library: it loads, exports every symbol the header declares, and its
host-only queries behave like the reference's (no GPU work here)."""
import os
import re
import subprocess
import sys

import numpy as np
import pytest

import ruquant_amd as rq
from ruquant_amd.lib import PROTOTYPES, LIB_PATH, ABI_VERSION, PROBE_PATH

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "rq_w4a4.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rq_w4a4_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = rq.load_library()
    syms = header_symbols()
    assert len(syms) >= 12
    for s in syms:
        assert hasattr(L, s), s
        assert s in PROTOTYPES, "python binding lacks %s" % s
    assert L.rq_w4a4_abi_version() == ABI_VERSION
    header = open(os.path.join(ROOT, "include", "rq_w4a4.h")).read()
    assert int(re.search(r"#define RQ_ABI_VERSION (\d+)", header).group(1)) == ABI_VERSION


def test_probe_library_exports_its_header():
    text = open(os.path.join(ROOT, "include", "rq_probe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    syms = sorted(set(re.findall(r"\b(rq_probe\w*)\s*\(", text)))
    assert syms == ["rq_probe"]
    P = rq.load_probe_library()
    assert hasattr(P, "rq_probe")
    assert os.path.exists(PROBE_PATH) and PROBE_PATH.startswith(ROOT)
    # the operator's library carries no measurement kernels
    assert not hasattr(rq.load_library(), "rq_probe") and not hasattr(rq.load_library(), "rq_w4a4_probe")


def test_stage_mask_is_a_host_query():
    L = rq.load_library()
    assert L.rq_w4a4_stage_mask(rq.TYPE_W4A4H, 5120, 1, 5120) in (2, 3)   # (3 under RQ_DECODE_FUSED=0 / RQ_ACT_GROUP)
    assert L.rq_w4a4_stage_mask(rq.TYPE_W4A4H, 17408, 1, 17408) == 3       # H68: two launches at one token
    assert L.rq_w4a4_stage_mask(rq.TYPE_W4A4H, 5120, 2, 5120) == 3
    assert L.rq_w4a4_stage_mask(rq.TYPE_W4A4, 4096, 512, 4096) == 3
    assert L.rq_w4a4_stage_mask(12, 4096, 1, 4096) == 0
    assert L.rq_w4a4_stage_mask(rq.TYPE_W4A4H, 5120, 1, 1000) == 0


def test_library_is_in_tree():
    assert os.path.exists(LIB_PATH) and LIB_PATH.startswith(ROOT)


def test_hadamard_factor_matches_oracle(oracle):
    for n in [1, 12, 20, 64, 128, 256, 512, 768, 1024, 1536, 4096, 4352, 5120, 6144, 17408, 32768, 1792, 7 * 256,
              44 * 64, 60 * 32, 72 * 64, 84 * 4, 104 * 16, 108 * 256, 24 * 8, 36 * 4]:
        assert rq.hadamard_factor(n) == oracle.hadamard_factor(n), n


def test_supported_mirrors_reference_rules():
    assert rq.supported(rq.TYPE_W4A4H, 5120, 17408, 1)
    assert rq.supported(rq.TYPE_W4A4, 4096, 1024, 1)
    assert not rq.supported(rq.TYPE_W4A4, 4096 + 128, 1024, 1)      # K % 256
    assert not rq.supported(rq.TYPE_W4A4, 32768 + 256, 1024, 1)     # K <= 32768
    assert not rq.supported(rq.TYPE_W4A4H, 7 * 256, 1024, 1)        # no Hadamard factorization
    assert rq.supported(rq.TYPE_W4A4, 7 * 256, 1024, 1)
    assert not rq.supported(rq.TYPE_W4A4, 4096, 1024, 4, ldx_bytes=4096 * 4 + 4)   # row stride % 16
    assert not rq.supported(12, 4096, 1024, 1)                      # another ggml type
    assert rq.supported(rq.TYPE_W4A4, 256, 136, 3)                  # any N (the reference needs N % 64 == 0)


def test_sizes_are_aligned_and_monotone():
    L = rq.load_library()
    assert L.rq_w4a4_prepared_bytes(5120, 17408) % 256 == 0
    assert L.rq_w4a4_prepared_bytes(5120, 17408) >= 5120 * 17408 // 2
    assert L.rq_w4a4_prepared_bytes(100, 8) == 0
    a = L.rq_w4a4_workspace_bytes(rq.TYPE_W4A4H, 5120, 17408, 1)
    b = L.rq_w4a4_workspace_bytes(rq.TYPE_W4A4H, 5120, 17408, 2048)
    assert a % 256 == 0 and b % 256 == 0 and b > a > 0


def test_mul_mat_rejects_bad_arguments_without_touching_the_gpu():
    L = rq.load_library()
    assert L.rq_w4a4_mul_mat(rq.TYPE_W4A4, None, 4096, 1024, None, 4096, 1, None, 1024, 1.0, 0, None, 0, None) == -3
    assert L.rq_w4a4_prepare(None, 4096, 1024, None, 0, None) == -3
    assert L.rq_w4a4_prepare(1 << 20, 100, 1024, 1 << 20, 1 << 30, None) == -1


def _clip_in_subprocess(env, pad1, type_):
    code = (
        "import numpy as np, ruquant_amd as rq\n"
        "b = np.zeros(1, dtype=rq.BLOCK_DTYPE)\n"
        "b['pad'][0, 1] = np.float32(%r).view(np.int32)\n"
        "print(repr(rq.resolve_clip(b[0], %d)))\n" % (pad1, type_))
    e = dict(os.environ)
    e.pop("RQ_ACT_CLIP", None)
    e.pop("RQ_ACT_CLIP_H", None)
    e.update(env)
    out = subprocess.run([sys.executable, "-c", code], cwd=ROOT, env=e, capture_output=True, text=True, check=True)
    return float(out.stdout.strip())


def test_clip_precedence_env_then_header_then_one():
    f = lambda v: float(np.float32(v))
    assert _clip_in_subprocess({}, 0.0, rq.TYPE_W4A4) == 1.0
    assert _clip_in_subprocess({}, 0.9, rq.TYPE_W4A4H) == f(0.9)
    assert _clip_in_subprocess({"RQ_ACT_CLIP_H": "0.85"}, 0.9, rq.TYPE_W4A4H) == f(0.85)
    assert _clip_in_subprocess({"RQ_ACT_CLIP_H": "0.85"}, 0.9, rq.TYPE_W4A4) == f(0.9)   # _H does not reach W4A4
    assert _clip_in_subprocess({"RQ_ACT_CLIP": "0.8"}, 0.9, rq.TYPE_W4A4H) == f(0.8)     # plain one reaches both
    assert _clip_in_subprocess({"RQ_ACT_CLIP": "0.8", "RQ_ACT_CLIP_H": "0.7"}, 0.0, rq.TYPE_W4A4H) == f(0.7)
    assert _clip_in_subprocess({"RQ_ACT_CLIP": "-1"}, 0.0, rq.TYPE_W4A4) == 1.0


def test_tensor_rot():
    b = np.zeros(1, dtype=rq.BLOCK_DTYPE)
    b["pad"][0, 0] = 5120
    assert rq.tensor_rot(b[0], rq.TYPE_W4A4H, 5120) == 5120
    assert rq.tensor_rot(b[0], rq.TYPE_W4A4H, 10240) == 5120
    assert rq.tensor_rot(b[0], rq.TYPE_W4A4H, 6144) == -1    # does not divide
    assert rq.tensor_rot(b[0], rq.TYPE_W4A4, 6144) == 0
    b["pad"][0, 0] = 7 * 256
    assert rq.tensor_rot(b[0], rq.TYPE_W4A4H, 7 * 256) == -1  # no factorization
    b["pad"][0, 0] = 0
    assert rq.tensor_rot(b[0], rq.TYPE_W4A4H, 4096) == -1


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    import ruquant_amd.lib as lib
    monkeypatch.setattr(lib, "_lib", None)
    monkeypatch.setattr(lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(lib.LibraryMissing):
        lib.load_library()
