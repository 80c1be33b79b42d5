"""fp32 CPU restatements of the hot-path arithmetic (test infrastructure).

Reference call sites these restate:
  gemm              include/kernels/gemm_device.cuh:110-169, oracle of tests/python/test_gemm.py:55
  fused_two_gemms   include/kernels/fused_two_gemms_device.cuh:114-214,
                    oracle of tests/python/test_fused_two_gemms.py:100
  flash_attention   include/kernels/flash_attention_device.cuh:130-312 (mask: include/cell/mask.hpp:75-82),
                    blockwise oracle tests/python/test_flash_attn.py:85-134
  flash_decode      no reference counterpart (split-KV + log-sum-exp combine, closed form)
"""

import math

import torch

REL_L2_TOL = 1e-3
MAX_ABS_TOL = 2e-2


def rel_l2(y: torch.Tensor, ref: torch.Tensor) -> float:
    y = y.detach().double().cpu()
    ref = ref.detach().double().cpu()
    return float((y - ref).norm() / ref.norm().clamp_min(1e-30))


def max_abs(y: torch.Tensor, ref: torch.Tensor) -> float:
    return float((y.detach().double().cpu() - ref.detach().double().cpu()).abs().max())


def check_close(y, ref, rel_tol=REL_L2_TOL, abs_tol=MAX_ABS_TOL):
    """Return (ok, rel_l2, max_abs) under the tolerance the benchmark contract states."""
    r, a = rel_l2(y, ref), max_abs(y, ref)
    return (r <= rel_tol and a <= abs_tol and math.isfinite(r)), r, a


def gemm_ref(a: torch.Tensor, b_nk: torch.Tensor) -> torch.Tensor:
    """C[m,n] = sum_k A[m,k] * B[k,n]; B is handed over as its [n,k] buffer (col-major k x n)."""
    return a.float().cpu() @ b_nk.float().cpu().T


def fused_two_gemms_ref(a, b_nk, c_pn):
    """D = (A @ B) @ C with B as an [n,k] buffer and C as a [p,n] buffer, all fp32."""
    return (a.float().cpu() @ b_nk.float().cpu().T) @ c_pn.float().cpu().T


def fused_two_gemms_ref_rounded(a, b_nk, c_pn):
    """Same, with the intermediate rounded to fp16 like the kernel does
    (include/kernels/fused_two_gemms_device.cuh:200) - bounds the expected error."""
    p = (a.float().cpu() @ b_nk.float().cpu().T).half().float()
    return p @ c_pn.float().cpu().T


def attention_ref(q, k, v, scale=None, causal=False):
    """O = softmax(scale * Q K^T + mask) V over the last two dims; leading dims are batch.
    q [..., Lq, D], k [..., Lkv, D], v [..., Lkv, Dv].  Causal mask: col > row -> -inf
    (global coordinates, include/cell/mask.hpp:75-82)."""
    q, k, v = q.float().cpu(), k.float().cpu(), v.float().cpu()
    scale = 1.0 / math.sqrt(q.shape[-1]) if scale is None else scale
    s = (q @ k.transpose(-1, -2)) * scale
    if causal:
        lq, lkv = s.shape[-2], s.shape[-1]
        row = torch.arange(lq).unsqueeze(-1)
        col = torch.arange(lkv).unsqueeze(0)
        s = s.masked_fill(col > row, float("-inf"))
    p = torch.softmax(s, dim=-1)
    return p @ v


def attention_blockwise_ref(q, k, v, tile_kv, scale=None, causal=False):
    """Blockwise online-softmax restatement of tests/python/test_flash_attn.py:85-134 for a
    single [Lq, D] x [Lkv, D] x [Lkv, Dv] problem, in fp32, with the running maximum started
    at -inf and the causal mask in global coordinates (the reference starts at 0 and masks
    chunk-locally, which is only right for one KV chunk)."""
    q, k, v = q.float().cpu(), k.float().cpu(), v.float().cpu()
    scale = 1.0 / math.sqrt(q.shape[-1]) if scale is None else scale
    lq, lkv = q.shape[0], k.shape[0]
    out = torch.zeros(lq, v.shape[1])
    prev_max = torch.full((lq, 1), float("-inf"))
    prev_sum = torch.zeros(lq, 1)
    row = torch.arange(lq).unsqueeze(-1)
    for start in range(0, lkv, tile_kv):
        kc, vc = k[start:start + tile_kv], v[start:start + tile_kv]
        s = (q @ kc.T) * scale
        if causal:
            col = torch.arange(start, start + kc.shape[0]).unsqueeze(0)
            s = s.masked_fill(col > row, float("-inf"))
        cur_max = s.max(dim=-1, keepdim=True).values
        new_max = torch.maximum(cur_max, prev_max)
        safe_max = torch.where(torch.isinf(new_max), torch.zeros_like(new_max), new_max)
        e = torch.exp(s - safe_max)
        renorm_prev = torch.exp(prev_max - safe_max)
        new_sum = renorm_prev * prev_sum + e.sum(dim=-1, keepdim=True)
        out = out * renorm_prev + e @ vc
        prev_max, prev_sum = new_max, new_sum
    return out / prev_sum


def flash_decode_ref(q, k, v, scale=None):
    """Single-query attention. q [..., D], k [..., Lkv, D], v [..., Lkv, Dv] -> [..., Dv]."""
    q, k, v = q.float().cpu(), k.float().cpu(), v.float().cpu()
    scale = 1.0 / math.sqrt(q.shape[-1]) if scale is None else scale
    s = (k @ q.unsqueeze(-1)).squeeze(-1) * scale
    p = torch.softmax(s, dim=-1)
    return (p.unsqueeze(-2) @ v).squeeze(-2)


def split_kv_partials(q, k, v, num_splits, scale=None):
    """Per-split partial results of single-query attention for one (batch, head) slice:
    o_s [num_splits, Dv] (un-normalised, relative to m_s), m_s [num_splits], l_s [num_splits]."""
    q, k, v = q.float().cpu(), k.float().cpu(), v.float().cpu()
    scale = 1.0 / math.sqrt(q.shape[-1]) if scale is None else scale
    lkv = k.shape[0]
    chunk = (lkv + num_splits - 1) // num_splits
    o, m, l = [], [], []
    for s in range(num_splits):
        kc, vc = k[s * chunk:(s + 1) * chunk], v[s * chunk:(s + 1) * chunk]
        if kc.shape[0] == 0:
            o.append(torch.zeros(v.shape[1])); m.append(torch.tensor(float("-inf"))); l.append(torch.tensor(0.0))
            continue
        sc = (kc @ q) * scale
        ms = sc.max()
        e = torch.exp(sc - ms)
        o.append(e @ vc); m.append(ms); l.append(e.sum())
    return torch.stack(o), torch.stack(m), torch.stack(l)


def combine_partials(o, m, l):
    """O = sum_s e^{m_s-M} o_s / sum_s e^{m_s-M} l_s with M = max_s m_s."""
    big = m.max()
    w = torch.exp(m - big)
    return (w.unsqueeze(-1) * o).sum(dim=0) / (w * l).sum()


def scatter_nd_ref(data, indices, updates):
    """data[indices[i]] += updates[i] for every index row (duplicates accumulate), fp32 on the
    CPU.  Restates what ke_scatter_nd computes (src/kernels/scatter_nd.cu:10-34) with the
    library routine torch.Tensor.index_put_(accumulate=True)."""
    out = data.detach().float().cpu().clone()
    idx = indices.detach().cpu().long()
    k = idx.shape[-1]
    idx = idx.reshape(-1, k)
    upd = updates.detach().float().cpu().reshape(idx.shape[0], *out.shape[k:])
    out.index_put_(tuple(idx[:, j] for j in range(k)), upd, accumulate=True)
    return out
