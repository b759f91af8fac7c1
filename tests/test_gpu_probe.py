"""The measurement probes of librq_probe.so (rq_probe): every kind launches and returns, and its argument checks
refuse what the kernels cannot take. What they measure is bench.py's business (`extra.peaks`)."""
import pytest
import torch

import ruquant_amd as rq

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
EMPTY, STREAM, MIX = 0, 1, 2


def _probe(L, buf, kind, a0, a1=0, a2=0, a3=0, nbytes=None):
    stream = torch.cuda.current_stream().cuda_stream
    return L.rq_probe(kind, a0, a1, a2, a3, buf.data_ptr(), buf.numel() if nbytes is None else nbytes, stream)


def test_probe_kinds_launch_and_return():
    L = rq.load_probe_library()
    buf = torch.ones(1 << 22, dtype=torch.uint8, device=DEV)
    assert _probe(L, buf, EMPTY, 256) == 0
    for loads in (4, 5, 8, 10, 16, 20):
        assert _probe(L, buf, STREAM, loads * 4096 * 16, loads, 0) == 0
    assert _probe(L, buf, STREAM, 1 << 22, 8, 64) == 0
    for sub in range(8):
        for op in range(6):
            assert _probe(L, buf, MIX, sub | op << 8, 4, 2, 2) == 0
        for form in (1, 2, 3):   # the other MFMA forms, beside v_add_u32 and v_fma_f32
            for op in (0, 4):
                assert _probe(L, buf, MIX, sub | op << 8 | form << 20, 4, 2, 2) == 0
    assert _probe(L, buf, MIX, 5 | 1 << 16, 4, 2, 2) == 0
    assert _probe(L, buf, MIX, 0, 4, 2, 2) == 0
    torch.cuda.synchronize()
    # workgroup 0 reports the SIMD of each of its eight wavefronts: all four SIMDs of the compute unit are used
    simds = buf[4096:4096 + 32].view(torch.int32).cpu().tolist()
    assert all(0 <= v <= 3 for v in simds) and set(simds) == {0, 1, 2, 3}, simds


def test_probe_argument_checks():
    L = rq.load_probe_library()
    buf = torch.ones(1 << 20, dtype=torch.uint8, device=DEV)
    assert _probe(L, buf, 9, 1) != 0                           # unknown kind
    assert _probe(L, buf, EMPTY, 0) != 0                       # no workgroups
    assert _probe(L, buf, STREAM, 1 << 20, 7, 0) != 0          # loads in flight not one of the built counts
    assert _probe(L, buf, STREAM, 1 << 21, 8, 0) != 0          # more bytes than the buffer holds
    assert _probe(L, buf, STREAM, 12345, 8, 0) != 0            # not whole chunks
    assert _probe(L, buf, MIX, 8, 4, 2, 2) != 0                # unknown sub-kind
    assert _probe(L, buf, MIX, 0 | 6 << 8, 4, 2, 2) != 0       # unknown VALU instruction
    assert _probe(L, buf, MIX, 0 | 2 << 8 | 3 << 20, 4, 2, 2) != 0   # a combination that is not built
    assert _probe(L, buf, MIX, 0, 0, 2, 2) != 0                # no workgroups
    assert _probe(L, buf, EMPTY, 256, nbytes=1024) != 0        # scratch too small
    torch.cuda.synchronize()
