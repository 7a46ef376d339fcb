"""Weighted flash decoding and the estimation zone.

The reference calls an external fork (see the package docstring: parity unpinned); the
arithmetic below is the one its call sites imply
(cache_hub/retroinfer_cache.py:611-617 estimation call, :666-674 final call):

    out = (e^{lse_prev} * out_prev + sum_r e^{s_r} v_r) / (e^{lse_prev} + sum_r w_r e^{s_r})
    lse = log(denominator),  s_r = scale * q.k_r

Computed in fp64 from the 16-bit inputs; outputs rounded to their element type like the kernel's.
"""
import math
import torch


def weighted_flash_decoding(q, k, v, weight=None, previous_out=None, previous_lse=None,
                            cache_seqlens=None, scale=None):
    """q [BG, gs, D]; k, v [BG, S, D]; weight [BG, S] or None; previous_out [BG, gs, D] and
    previous_lse [BG, gs] or None; cache_seqlens [BG] or None.  Returns (out bf16, lse fp32)."""
    BG, gs, D = q.shape
    S = k.shape[1]
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    out = torch.empty(BG, gs, D, dtype=q.dtype if q.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16)
    lse = torch.empty(BG, gs, dtype=torch.float32)
    for g in range(BG):
        n = S if cache_seqlens is None else int(cache_seqlens[g])
        s = (q[g].double() @ k[g, :n].double().T) * scale          # [gs, n]
        w = torch.ones(n, dtype=torch.float64) if weight is None else weight[g, :n].double()
        m = s.max(dim=-1).values if n > 0 else torch.full((gs,), -math.inf, dtype=torch.float64)
        if previous_lse is not None:
            m = torch.maximum(m, previous_lse[g].double())
        p = torch.exp(s - m[:, None])
        num = p @ v[g, :n].double()
        den = (p * w[None, :]).sum(-1)
        if previous_lse is not None:
            f = torch.exp(previous_lse[g].double() - m)
            num = num + f[:, None] * previous_out[g].double()
            den = den + f
        out[g] = (num / den[:, None]).to(out.dtype)
        lse[g] = (m + torch.log(den)).to(torch.float32)
    return out, lse


def estimation(logits, est_ids, value_sum, cluster_size_bf16):
    """Estimation-zone partial from the scoring logits (the call at
    cache_hub/retroinfer_cache.py:611-617, semantics inferred from its operands): scores are the
    cluster logits s_i = q.c_i / sqrt(D), values the cluster value sums, the denominator weights
    e^{s_i} by the bf16 cluster sizes: out = sum_i e^{s_i} VS_i / sum_i w_i e^{s_i},
    lse = log sum_i w_i e^{s_i}.
    logits [BG, gs, nc] fp32, est_ids [BG, es].  Returns (es_out fp64 [BG, gs, D], lse fp64)."""
    BG, gs, nc = logits.shape
    D = value_sum.shape[-1]
    out = torch.empty(BG, gs, D, dtype=torch.float64)
    lse = torch.empty(BG, gs, dtype=torch.float64)
    for g in range(BG):
        ids = est_ids[g].long()
        s = logits[g][:, ids].double()
        w = cluster_size_bf16[g, ids].double()
        m = s.max(-1).values
        p = torch.exp(s - m[:, None])
        den = (p * w[None, :]).sum(-1)
        out[g] = (p @ value_sum[g, ids].double()) / den[:, None]
        lse[g] = m + torch.log(den)
    return out, lse
