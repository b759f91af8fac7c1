"""Host-side mirror of the reference's W4A4 operator interface over the C ABI.

Names follow the reference's backend entry points (patches/llama.cpp-ruquant.patch, rq-w4a4.cuh, lines
2391-2401 of the patch): ``supported`` <-> ggml_cuda_rq_w4a4_supported, ``W4A4Weight.ready`` <->
ggml_cuda_rq_w4a4_ready, ``mul_mat`` <-> ggml_cuda_mul_mat_rq_w4a4, ``mul_mat_fused`` <->
ggml_cuda_mul_mat_rq_w4a4_fused. A ``W4A4Weight`` plays the part of the ggml weight tensor plus the
``rq_tensor_info`` the reference hangs on ``src0->extra`` at first use (patch lines 2027-2043).

torch owns device memory and the stream; every computation happens inside librq_w4a4.so.
"""
import ctypes

import numpy as np
import torch

from .lib import load_library

TYPE_W4A4, TYPE_W4A4H, TYPE_A4, TYPE_A4H = 44, 45, 46, 47
BLOCK_DTYPE = np.dtype([("d", "<f4"), ("sum", "<i4"), ("pad", "<i4", (2,)), ("qs", "<u4", (32,))])


class RqError(RuntimeError):
    pass


_ERRORS = {-1: "unsupported shape or type", -2: "workspace / prepared buffer too small or misaligned",
           -3: "bad argument"}


def _check(rc, what):
    if rc != 0:
        raise RqError("%s failed: %s" % (what, _ERRORS.get(rc, "hipError_t %d" % rc)))


def _stream_ptr():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _device_bytes(n, device):
    # torch's caching allocator returns 512-byte aligned blocks; the ABI needs 256
    t = torch.empty(max(int(n), 256), dtype=torch.uint8, device=device)
    assert t.data_ptr() % 256 == 0
    return t


def hadamard_factor(n):
    p, m = ctypes.c_int(0), ctypes.c_int(0)
    ok = load_library().rq_w4a4_hadamard_factor(int(n), ctypes.byref(p), ctypes.byref(m))
    return (p.value, m.value) if ok else None


def supported(type_, K, N, M, ldx_bytes=None, ldy_bytes=None):
    ldx_bytes = 4 * K if ldx_bytes is None else ldx_bytes
    ldy_bytes = 4 * N if ldy_bytes is None else ldy_bytes
    return bool(load_library().rq_w4a4_supported(type_, K, N, M, ldx_bytes, ldy_bytes))


def resolve_clip(block0, type_):
    """block0: the first block of the tensor (numpy, host). Environment > header pad[1] > 1."""
    b = np.ascontiguousarray(block0).view(np.uint8)
    return float(load_library().rq_w4a4_resolve_clip(b.ctypes.data, type_))


def tensor_rot(block0, type_, K):
    b = np.ascontiguousarray(block0).view(np.uint8)
    return int(load_library().rq_w4a4_tensor_rot(b.ctypes.data, type_, K))


class W4A4Weight:
    """A W4A4 / W4A4H weight tensor on the GPU: [N, K/256] blocks as ggml stores them, plus what the first use
    derives (clip, Hadamard length, the prepared streaming form)."""

    def __init__(self, blocks, type_, device="cuda:0", keep_blocks=True, in_place=False):
        blocks = np.ascontiguousarray(blocks)
        assert blocks.dtype == BLOCK_DTYPE and blocks.ndim == 2
        self.type = int(type_)
        self.N, nb = blocks.shape
        self.K = nb * 256
        self.device = torch.device(device)
        L = load_library()
        # first use: header of block 0 (the reference reads it back from the device, patch lines 2030-2040)
        self.clip = resolve_clip(blocks[0, 0], self.type)
        self.n_rot = tensor_rot(blocks[0, 0], self.type, self.K)
        if self.type == TYPE_W4A4H and self.n_rot < 0:
            raise RqError("W4A4H: Hadamard length %d does not divide this row of %d"
                          % (int(blocks[0, 0]["pad"][0]), self.K))
        b0 = np.ascontiguousarray(blocks[0, 0]).view(np.uint8)
        if L.rq_w4a4_weight_group(b0.ctypes.data) == 64 and L.rq_w4a4_act_group() != 64:
            # the reference asserts the same in ggml_vec_dot_w4a4_a4 (patch lines 169-170)
            raise RqError("weight groups of 64 need activation groups of 64 (RQ_ACT_GROUP=%d)" % L.rq_w4a4_act_group())
        raw = torch.from_numpy(blocks.view(np.uint8).reshape(-1).copy()).to(self.device)
        nbytes = L.rq_w4a4_prepared_bytes(self.K, self.N)
        if nbytes == 0:
            raise RqError("unsupported weight shape K=%d N=%d" % (self.K, self.N))
        self.plane6 = None
        if in_place:
            # as the reference repacks (patch lines 2046-2075): the tensor's own buffer becomes the prepared weight
            # (one copy of the codes resident), the fp6 plane of the wide-batch kernel lives beside it
            n6 = L.rq_w4a4_plane6_bytes(self.K, self.N)
            self.plane6 = _device_bytes(n6, self.device) if n6 else None
            staging = _device_bytes(L.rq_w4a4_inplace_staging_bytes(self.K, self.N), self.device)
            with torch.cuda.device(self.device):
                _check(L.rq_w4a4_prepare_inplace(raw.data_ptr(), self.K, self.N,
                                                 self.plane6.data_ptr() if n6 else None, n6, staging.data_ptr(),
                                                 staging.numel(), _stream_ptr()), "rq_w4a4_prepare_inplace")
                torch.cuda.current_stream().synchronize()   # staging is released below
            self.prepared = raw
            self.blocks = None
        else:
            self.prepared = _device_bytes(nbytes, self.device)
            with torch.cuda.device(self.device):
                _check(L.rq_w4a4_prepare(raw.data_ptr(), self.K, self.N, self.prepared.data_ptr(), nbytes,
                                         _stream_ptr()), "rq_w4a4_prepare")
            self.blocks = raw if keep_blocks else None
        self.ready = True

    def workspace(self, M):
        n = load_library().rq_w4a4_workspace_bytes(self.type, self.K, self.N, M)
        return _device_bytes(n, self.device)


def mul_mat(weight, x, out=None, workspace=None, clip=None):
    """y[M, N] = x[M, K] . W^T, bit-identical to the ggml-cpu W4A4 / W4A4H MUL_MAT."""
    return mul_mat_fused([weight], x, outs=None if out is None else [out], workspace=workspace, clip=clip)[0]


def fused_workspace_bytes(weights, M):
    """Workspace for a fused call that serves all its weights from one launch of the streaming kernels: split-K
    cells for the rows of every weight (each padded to 64). With room for the largest weight only
    (rq_w4a4_workspace_bytes of the largest N) the call still works, one product launch per weight."""
    w0 = weights[0]
    N = w0.N if len(weights) == 1 else sum((w.N + 63) // 64 * 64 for w in weights)
    return load_library().rq_w4a4_workspace_bytes(w0.type, w0.K, N, M)


def mul_mat_fused(weights, x, outs=None, workspace=None, clip=None):
    """Up to three weights of one type, K, clip and rotation length against the same activations."""
    L = load_library()
    w0 = weights[0]
    assert x.is_cuda and x.dtype == torch.float32 and x.dim() == 2 and x.stride(1) == 1
    M, K = x.shape
    assert K == w0.K
    for w in weights[1:]:
        if (w.type, w.K, w.clip, w.n_rot) != (w0.type, w0.K, w0.clip, w0.n_rot):
            raise RqError("weights cannot be fused: type, K, clip and rotation length must match")
    if outs is None:
        outs = [torch.empty((M, w.N), dtype=torch.float32, device=x.device) for w in weights]
    n = len(weights)
    if workspace is None:
        workspace = _device_bytes(fused_workspace_bytes(weights, M), x.device)
    prepared = (ctypes.c_void_p * n)(*[w.prepared.data_ptr() for w in weights])
    ys = (ctypes.c_void_p * n)(*[o.data_ptr() for o in outs])
    Ns = (ctypes.c_int64 * n)(*[w.N for w in weights])
    ldys = (ctypes.c_int64 * n)(*[o.stride(0) if o.shape[0] > 1 else o.shape[1] for o in outs])
    ldx = x.stride(0) if M > 1 else K
    with torch.cuda.device(x.device):
        rc = L.rq_w4a4_mul_mat_fused(w0.type, n, prepared, K, Ns, x.data_ptr(), ldx, M, ys, ldys,
                                     w0.clip if clip is None else clip, max(w0.n_rot, 0),
                                     workspace.data_ptr(), workspace.numel(), _stream_ptr())
    _check(rc, "rq_w4a4_mul_mat")
    return outs


class SharedActivation:
    """The reference's rq_act_cache (patch lines 1996-2023, 2160-2172) for this host: consecutive MUL_MATs of one x
    that were not fused rotate and quantize x once. The cache is the workspace itself; `begin()` plays
    ggml_cuda_rq_graph_begin (x may have changed in place since the last evaluation)."""

    def __init__(self, workspace):
        self.workspace = workspace
        workspace.zero_()            # the split-K cells inside must read zero before stage 2 first uses them
        self.key = None
        self.rows_cleared = 0
        self.hits = self.misses = 0

    def begin(self):
        self.key = None

    def mul_mat(self, weight, x, out):
        L = load_library()
        M, K = x.shape
        key = (x.data_ptr(), x.stride(0), M, K, weight.type, weight.clip, weight.n_rot)
        rows = (weight.N + 63) // 64 * 64
        hit = key == self.key and rows <= self.rows_cleared
        ldx = x.stride(0) if M > 1 else K
        ldy = out.stride(0) if M > 1 else weight.N
        with torch.cuda.device(x.device):
            rc = L.rq_w4a4_mul_mat_stages(weight.type, weight.prepared.data_ptr(), K, weight.N, x.data_ptr(), ldx, M,
                                          out.data_ptr(), ldy, weight.clip, max(weight.n_rot, 0),
                                          self.workspace.data_ptr(), self.workspace.numel(), _stream_ptr(),
                                          2 if hit else 3)
        _check(rc, "rq_w4a4_mul_mat_stages")
        if hit:
            self.hits += 1
        else:
            self.misses += 1
            self.key, self.rows_cleared = key, rows
        return out


def hadamard(x, n_rot=None):
    """x[M, K] -> x diag(H, H, ...) with H of length n_rot (default K), as ggml_rq_hadamard does per block."""
    L = load_library()
    assert x.is_cuda and x.dtype == torch.float32 and x.dim() == 2 and x.stride(1) == 1
    M, K = x.shape
    out = torch.empty((M, K), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        rc = L.rq_w4a4_hadamard(x.data_ptr(), x.stride(0) if M > 1 else K, M, K, n_rot or K, out.data_ptr(), K,
                                _stream_ptr())
    _check(rc, "rq_w4a4_hadamard")
    return out


def quantize_act(x, clip, hadamard_=False, n_rot=None):
    """x[M, K] -> [M, K/256] activation blocks in the reference's A4 / A4H layout (numpy, host)."""
    L = load_library()
    assert x.is_cuda and x.dtype == torch.float32 and x.dim() == 2 and x.stride(1) == 1
    M, K = x.shape
    out = torch.zeros(M * (K // 256) * 144, dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        rc = L.rq_w4a4_quantize_act(TYPE_A4H if hadamard_ else TYPE_A4, x.data_ptr(), x.stride(0) if M > 1 else K,
                                    M, K, clip, (n_rot or K) if hadamard_ else 0, out.data_ptr(), _stream_ptr())
    _check(rc, "rq_w4a4_quantize_act")
    return out.cpu().numpy().view(BLOCK_DTYPE).reshape(M, K // 256)


def quantize_weights(w, type_, n_rot=None, wgroup=0):
    """w[N, K] fp32 on the GPU -> [N, K/256] weight blocks (numpy, host): the type's from_float_ref for whole
    tensors (quantize_row_w4a4_ref / quantize_row_w4a4h_ref, patch lines 2681-2710). wgroup 0 / 256 / 64 is the
    reference's RQ_WGROUP switch; n_rot (W4A4H) its K / RQ_ROT_BLOCKS, default K."""
    L = load_library()
    assert w.is_cuda and w.dtype == torch.float32 and w.dim() == 2 and w.stride(1) == 1
    N, K = w.shape
    n_rot = int(n_rot or K)
    nbytes = L.rq_w4a4_quantize_weights_workspace_bytes(int(type_), K, N, int(wgroup))
    if nbytes == 0:
        raise RqError("unsupported weight shape or group: K=%d N=%d wgroup=%d" % (K, N, wgroup))
    ws = _device_bytes(nbytes, w.device)
    out = torch.zeros(N * (K // 256) * 144, dtype=torch.uint8, device=w.device)
    with torch.cuda.device(w.device):
        rc = L.rq_w4a4_quantize_weights(int(type_), w.data_ptr(), w.stride(0) if N > 1 else K, N, K, n_rot,
                                        int(wgroup), out.data_ptr(), ws.data_ptr(), ws.numel(), _stream_ptr())
    _check(rc, "rq_w4a4_quantize_weights")
    return out.cpu().numpy().view(BLOCK_DTYPE).reshape(N, K // 256)


def dequantize(blocks, type_, n_rot=None, device="cuda:0"):
    """[rows, K/256] blocks of any of the four types (numpy, host) -> [rows, K] fp32 on the GPU: the type's to_float
    (dequantize_row_w4a4 / _w4a4h / _a4 / _a4h, patch lines 2738-2773). The rotation length of the rotated types
    comes from block 0 (pad[0] of weights, pad[1] of activations) unless given."""
    L = load_library()
    blocks = np.ascontiguousarray(blocks)
    assert blocks.dtype == BLOCK_DTYPE and blocks.ndim == 2
    rows, nb = blocks.shape
    K = nb * 256
    if n_rot is None:
        n_rot = int(blocks[0, 0]["pad"][0 if type_ in (TYPE_W4A4, TYPE_W4A4H) else 1]) if rows else K
    dev = torch.device(device)
    raw = torch.from_numpy(blocks.view(np.uint8).reshape(-1).copy()).to(dev)
    out = torch.empty((rows, K), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        rc = L.rq_w4a4_dequantize(int(type_), raw.data_ptr(), rows, K, int(n_rot), out.data_ptr(), K, _stream_ptr())
    _check(rc, "rq_w4a4_dequantize")
    return out


# ---- on-disk format tools (host memory; the converter side of the reference) ----------------------------------

def pack(codes, scales):
    """int4 codes [N, K] (int8, -8..7) and one scale per row -> blocks [N, K/256] (src/gptq.rs:210-231 `pack`)."""
    codes = np.ascontiguousarray(codes, dtype=np.int8)
    scales = np.ascontiguousarray(scales, dtype=np.float32)
    N, K = codes.shape
    assert scales.shape == (N,)
    out = np.zeros((N, K // 256), dtype=BLOCK_DTYPE)
    _check(load_library().rq_w4a4_pack(codes.ctypes.data, scales.ctypes.data, N, K, out.ctypes.data), "rq_w4a4_pack")
    return out


def pack_groups(codes, units, mults):
    """As pack, with integer weight multipliers: mults [N, K/256] (per block) or [N, K/64] (per 64 inputs)
    (src/gptq.rs:193-207 `pack_groups`)."""
    codes = np.ascontiguousarray(codes, dtype=np.int8)
    units = np.ascontiguousarray(units, dtype=np.float32)
    mults = np.ascontiguousarray(mults, dtype=np.uint8)
    N, K = codes.shape
    per = mults.shape[1] // (K // 256)
    assert mults.shape == (N, per * (K // 256)) and per in (1, 4)
    out = np.zeros((N, K // 256), dtype=BLOCK_DTYPE)
    _check(load_library().rq_w4a4_pack_groups(codes.ctypes.data, units.ctypes.data, mults.ctypes.data, per, N, K,
                                              out.ctypes.data), "rq_w4a4_pack_groups")
    return out


def set_clip(blocks, clip):
    """Activation clip into pad[1] of every block, in place (`ruquant setclip`, src/convert.rs:876-878)."""
    assert blocks.dtype == BLOCK_DTYPE and blocks.flags.c_contiguous
    load_library().rq_w4a4_set_clip(blocks.ctypes.data, blocks.size, float(clip))


def set_rot_len(blocks, n):
    """Hadamard length into pad[0] of every block, in place (src/convert.rs:99-101 `set_rot_len`)."""
    assert blocks.dtype == BLOCK_DTYPE and blocks.flags.c_contiguous
    load_library().rq_w4a4_set_rot_len(blocks.ctypes.data, blocks.size, int(n))


def dequantize_rows(blocks):
    """The type's to_float for W4A4 weights: code * (multiplier * d) (patch lines 2738-2742). Returns [N, K] fp32."""
    assert blocks.dtype == BLOCK_DTYPE and blocks.ndim == 2 and blocks.flags.c_contiguous
    N, nb = blocks.shape
    out = np.empty((N, nb * 256), dtype=np.float32)
    _check(load_library().rq_w4a4_dequantize_rows(blocks.ctypes.data, N, nb * 256, out.ctypes.data),
           "rq_w4a4_dequantize_rows")
    return out
