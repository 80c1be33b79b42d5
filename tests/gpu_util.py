"""Helpers shared by the GPU parity tests: call the C ABI on torch device buffers."""

import math

import torch

from tilefusion_amd import _capi

DEV = "cuda:0"


def stream():
    return torch.cuda.current_stream().cuda_stream


def c_gemm(a, b, out_dtype=torch.float32, tiles=None, stages=1, level=0):
    lib = _capi.load()
    m, k = a.shape
    n = b.shape[0]
    tm, tn, tk = tiles if tiles else (m, n, k)
    c = torch.full((m, n), float("nan"), device=a.device, dtype=out_dtype)
    _capi.check(lib.tf_gemm_f16(a.data_ptr(), b.data_ptr(), c.data_ptr(), int(out_dtype == torch.float16),
                                m, n, k, tm, tn, tk, stages, level, stream()), "tf_gemm_f16")
    return c


def c_fused(a, b, c, tiles=None):
    lib = _capi.load()
    batch = 1 if a.dim() == 2 else a.shape[0]
    m, k = a.shape[-2:]
    n, p = b.shape[-2], c.shape[-2]
    tm, tn, tk, tp = tiles if tiles else (m, n, k, p)
    d = torch.full((*a.shape[:-1], p), float("nan"), device=a.device, dtype=torch.float16)
    _capi.check(lib.tf_fused_two_gemms_f16(a.data_ptr(), b.data_ptr(), c.data_ptr(), d.data_ptr(), batch,
                                           m, n, k, p, tm, tn, tk, tp, stream()), "tf_fused_two_gemms_f16")
    return d


def c_fused_dtype(a, b, c, tiles=None, workspace=False):
    """The dtype-coded entry points (fp16 or bf16 operands), without or with a workspace."""
    lib = _capi.load()
    batch = 1 if a.dim() == 2 else a.shape[0]
    m, k = a.shape[-2:]
    n, p = b.shape[-2], c.shape[-2]
    tm, tn, tk, tp = tiles if tiles else (m, n, k, p)
    code = _capi.TF_DTYPE_BF16 if a.dtype == torch.bfloat16 else _capi.TF_DTYPE_F16
    d = torch.full((*a.shape[:-1], p), float("nan"), device=a.device, dtype=a.dtype)
    if not workspace:
        _capi.check(lib.tf_fused_two_gemms(a.data_ptr(), b.data_ptr(), c.data_ptr(), d.data_ptr(), code, batch,
                                           m, n, k, p, tm, tn, tk, tp, stream()), "tf_fused_two_gemms")
        return d
    want = lib.tf_fused_two_gemms_workspace_bytes(code, batch, m, n, k, p)
    ws = torch.empty(max(want, 16), device=a.device, dtype=torch.uint8)
    _capi.check(lib.tf_fused_two_gemms_ws(a.data_ptr(), b.data_ptr(), c.data_ptr(), d.data_ptr(), code, batch, m, n, k, p,
                                          tm, tn, tk, tp, ws.data_ptr(), want, stream()), "tf_fused_two_gemms_ws")
    return d


def c_fused_ws(a, b, c, tiles=None, workspace_bytes=None):
    """The workspace form: returns (D, bytes the library asked for).  workspace_bytes overrides the
    size that is handed over (0: no workspace)."""
    lib = _capi.load()
    batch = 1 if a.dim() == 2 else a.shape[0]
    m, k = a.shape[-2:]
    n, p = b.shape[-2], c.shape[-2]
    tm, tn, tk, tp = tiles if tiles else (m, n, k, p)
    want = lib.tf_fused_two_gemms_workspace_bytes(_capi.TF_DTYPE_F16, batch, m, n, k, p)
    nbytes = want if workspace_bytes is None else workspace_bytes
    ws = torch.full((max(nbytes, 16),), 0xFF, device=a.device, dtype=torch.uint8)
    d = torch.full((*a.shape[:-1], p), float("nan"), device=a.device, dtype=torch.float16)
    _capi.check(lib.tf_fused_two_gemms_ws(a.data_ptr(), b.data_ptr(), c.data_ptr(), d.data_ptr(), _capi.TF_DTYPE_F16,
                                          batch, m, n, k, p, tm, tn, tk, tp, ws.data_ptr() if nbytes else None,
                                          nbytes, stream()), "tf_fused_two_gemms_ws")
    return d, want


def c_attention(q, k, v, causal=False, scale=None, v_transposed=False, tiles=None):
    """q [B, Lq, D], k [B, Lkv, D], v [B, Lkv, Dv] (or [B, Dv, Lkv] if v_transposed)."""
    lib = _capi.load()
    b, lq, d = q.shape
    lkv = k.shape[1]
    dv = v.shape[1] if v_transposed else v.shape[2]
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    t = tiles if tiles else (lq, lkv, d, dv)
    o = torch.full((b, lq, dv), float("nan"), device=q.device, dtype=q.dtype)
    if q.dtype == torch.bfloat16:   # the dtype-coded entry point: tuned bf16 kernels or the run-time compiled one
        _capi.check(lib.tf_flash_attention_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), _capi.TF_DTYPE_BF16,
                                               b, lq, lkv, d, dv, int(v_transposed), t[0], t[1], t[2], t[3], scale,
                                               int(causal), stream()), "tf_flash_attention_fwd")
        return o
    _capi.check(lib.tf_flash_attention_fwd_f16(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), b, lq, lkv,
                                               d, dv, int(v_transposed), t[0], t[1], t[2], t[3], scale, int(causal),
                                               stream()), "tf_flash_attention_fwd_f16")
    return o


def c_decode(q, k, v, num_splits, scale=None):
    """q [BH, D], k, v [BH, Lkv, D]; fp16 through tf_flash_decode_f16, bf16 through the dtype-coded entry."""
    lib = _capi.load()
    bh, lkv, d = k.shape
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    nbytes = lib.tf_flash_decode_workspace_bytes(bh, d, num_splits)
    ws = torch.empty(nbytes, device=q.device, dtype=torch.uint8)
    o = torch.full((bh, d), float("nan"), device=q.device, dtype=q.dtype)
    if q.dtype == torch.float16:
        _capi.check(lib.tf_flash_decode_f16(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), ws.data_ptr(), nbytes,
                                            bh, lkv, d, num_splits, scale, stream()), "tf_flash_decode_f16")
    else:
        _capi.check(lib.tf_flash_decode(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), 2, ws.data_ptr(), nbytes,
                                        bh, lkv, d, num_splits, scale, stream()), "tf_flash_decode")
    return o
