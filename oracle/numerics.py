"""Numerical restatements of the chunk-scheduled kernels on the CPU (oracle: test infrastructure).

  * ring_reduce          tests/test_gemm_rs.py:60-72 of the reference
  * gemm_fp32            syncopate/computation/gemm/template.py:139-157 (fp32 accumulate, one rounding)
  * chunked_attention    syncopate/computation/attn/template.py:173-349 (base-2 online softmax per
                         kv chunk, lse2 = m + log2(l), pairwise merge of (O, lse2) with O rounded to
                         the output type after every merge)
"""

from __future__ import annotations

from typing import Iterable, List, Optional, Sequence, Tuple

import numpy as np
import torch

LOG2E_REF = 1.44269504  # the literal the reference multiplies sm_scale by (attn/template.py:179)


# ------------------------------------------------------------------ 16-bit rounding in numpy

def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even fp32 -> bf16, returned as uint16 bit patterns (NaN kept quiet)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    out = rounded.astype(np.uint16)
    nan = np.isnan(x)
    if nan.any():
        out = np.where(nan, np.uint16(0x7FC0), out)
    return out


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def round_to(x: np.ndarray, dtype: str) -> np.ndarray:
    """fp32 values rounded to `dtype` ("bf16" | "fp16") and widened back to fp32."""
    if dtype == "bf16":
        return bf16_bits_to_f32(f32_to_bf16_bits(x))
    if dtype == "fp16":
        return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)
    raise ValueError(dtype)


# ------------------------------------------------------------------ ring reduce

def ring_reduce(recv: np.ndarray, local: np.ndarray, rank: int, *, dtype: str = "bf16",
                round_each_add: bool = True) -> np.ndarray:
    """out[m, n] = local[rank*Mr + m, n] + sum_{i=1..W-1} recv[(rank+i) % W, m, n], left to right.

    `recv` [W, Mr, N] and `local` [W*Mr, N] hold fp32 values that are exactly
    representable in `dtype`.  With round_each_add the running sum is rounded to
    `dtype` after every add (the reference accumulates in the tensor's dtype,
    tests/test_gemm_rs.py:64-70); otherwise it is kept in fp32 and rounded once.
    Returns fp32 values representable in `dtype`.
    """
    world, rows, _ = recv.shape
    acc = np.array(local[rank * rows:(rank + 1) * rows], dtype=np.float32, copy=True)
    for i in range(1, world):
        src = (rank + i) % world
        acc = acc + recv[src].astype(np.float32)
        if round_each_add:
            acc = round_to(acc, dtype)
    return round_to(acc, dtype)


# ------------------------------------------------------------------ GEMM

def gemm_fp32(a: torch.Tensor, b_nk: torch.Tensor) -> torch.Tensor:
    """C = A @ B^T in fp32 on the CPU; A [M, K], B stored [N, K] (template.py:53-58)."""
    return torch.matmul(a.detach().cpu().float(), b_nk.detach().cpu().float().t())


# ------------------------------------------------------------------ attention

def _partial_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, qk_scale: float,
                       block_n: int, p_dtype: torch.dtype,
                       mask: Optional[torch.Tensor]) -> Tuple[torch.Tensor, torch.Tensor]:
    """One program of the reference kernel: q [m, d] against k, v [n, d], base-2 online
    softmax over kv blocks of `block_n` (template.py:173-300).  Returns (O fp32 [m, d],
    lse2 fp32 [m]).  `mask` [m, n] True = keep."""
    m = q.shape[0]
    m_i = torch.full((m,), float("-inf"))
    l_i = torch.ones((m,))                      # the reference starts l at 1.0 (template.py:174)
    acc = torch.zeros((m, q.shape[1]))
    for lo in range(0, k.shape[0], block_n):
        kb, vb = k[lo:lo + block_n], v[lo:lo + block_n]
        qk = q @ kb.t()
        if mask is not None:
            qk = torch.where(mask[:, lo:lo + block_n], qk, torch.full_like(qk, float("-inf")))
        m_ij = torch.maximum(m_i, qk.max(dim=1).values * qk_scale)
        p = torch.exp2(qk * qk_scale - m_ij[:, None])
        alpha = torch.exp2(m_i - m_ij)
        l_i = l_i * alpha + p.sum(dim=1)
        acc = acc * alpha[:, None] + p.to(p_dtype).float() @ vb   # P is cast to the input type (:257)
        m_i = m_ij
    return acc / l_i[:, None], m_i + torch.log2(l_i)


def chunked_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    sm_scale: float,
    kv_chunks: Sequence[Tuple[int, int]],
    *,
    causal: bool = False,
    block_n: int = 128,
    round_merges: bool = True,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Attention of q [Z, H, Sq, D] over k, v [Z, H, Skv, D], the kv axis consumed as the
    element ranges `kv_chunks` in the given (arrival) order; each chunk yields a partial
    (O, lse2) that is merged into the running output exactly as the reference's epilogue
    does (template.py:328-349): the first partial is stored rounded to the output type,
    later ones are combined with m_new = max + log2(1 + 2^-|delta|) and the merged O is
    rounded to the output type again (round_merges=False keeps fp32 between merges).
    Returns (O in q's dtype, lse2 fp32 [Z, H, Sq]).
    """
    out_dtype = q.dtype
    qf, kf, vf = q.detach().cpu().float(), k.detach().cpu().float(), v.detach().cpu().float()
    Z, H, Sq, D = qf.shape
    qk_scale = float(np.float32(sm_scale) * np.float32(LOG2E_REF))
    o_run = torch.zeros((Z, H, Sq, D))
    lse_run = torch.zeros((Z, H, Sq))
    seen = torch.zeros((Z, H, Sq), dtype=torch.bool)
    rows = torch.arange(Sq)
    for lo, hi in kv_chunks:
        cols = torch.arange(lo, hi)
        mask = (cols[None, :] <= rows[:, None]) if causal else None
        for z in range(Z):
            for h in range(H):
                if causal:
                    live = mask.any(dim=1)             # q rows that see at least one kv of the chunk
                    if not live.any():
                        continue
                    o_p = torch.zeros((Sq, D))
                    l_p = torch.full((Sq,), float("-inf"))
                    o_live, l_live = _partial_attention(qf[z, h][live], kf[z, h, lo:hi], vf[z, h, lo:hi],
                                                        qk_scale, block_n, out_dtype, mask[live])
                    o_p[live], l_p[live] = o_live, l_live
                else:
                    live = torch.ones(Sq, dtype=torch.bool)
                    o_p, l_p = _partial_attention(qf[z, h], kf[z, h, lo:hi], vf[z, h, lo:hi],
                                                  qk_scale, block_n, out_dtype, None)
                first = live & ~seen[z, h]
                later = live & seen[z, h]
                if first.any():
                    o_run[z, h][first] = o_p[first]
                    lse_run[z, h][first] = l_p[first]
                if later.any():
                    m_old, m_new_part = lse_run[z, h][later], l_p[later]
                    delta = m_old - m_new_part
                    m_new = torch.maximum(m_old, m_new_part) + torch.log2(1.0 + torch.exp2(-delta.abs()))
                    w_old = torch.exp2(m_old - m_new)
                    w_part = torch.exp2(m_new_part - m_new)
                    o_run[z, h][later] = o_run[z, h][later] * w_old[:, None] + o_p[later] * w_part[:, None]
                    lse_run[z, h][later] = m_new
                seen[z, h] |= live
                if round_merges:
                    o_run[z, h] = o_run[z, h].to(out_dtype).float()
    return o_run.to(out_dtype), lse_run


def sdpa_fp32(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, sm_scale: float,
              causal: bool = False) -> torch.Tensor:
    """Library routine the chunked result must reduce to."""
    return torch.nn.functional.scaled_dot_product_attention(
        q.detach().cpu().float(), k.detach().cpu().float(), v.detach().cpu().float(),
        is_causal=causal, scale=sm_scale)
