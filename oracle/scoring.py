"""Centroid scoring and cluster selection.

Follows library/retroinfer/retroinfer_kernels/src/batch_gemm_softmax.cu:82-122 (alpha-scaled
GEMM, fp32 accumulate, bf16 D), batch_gemm_softmax.h:222-243 (softmax re-read from the bf16 D,
max/sum from the fp32 values) and cache_hub/retroinfer_cache.py:572-575 (sum over the query
group, empty-cluster mask, top-k).
"""
import math
import torch

from .numerics import rb, BF16_MIN


def logits_fp32(q: torch.Tensor, cent: torch.Tensor, scale: float) -> torch.Tensor:
    """x[g,j,c] = fp32(sum_d q*c) * scale.  The dot product is accumulated in fp64 and rounded
    once: the ideal of the reference's fp32 tensor-core accumulation, whose order is unspecified."""
    acc = torch.matmul(q.double(), cent.double().transpose(1, 2)).to(torch.float32)
    return acc * torch.tensor(scale, dtype=torch.float32)


def softmax_from_logits(x: torch.Tensor, dtype=torch.bfloat16):
    """(D, row max, 1/row sum, Softmax) from fp32 logits x [BG, gs, nc]; D and Softmax in the 16-bit element
    type of the operator's tensors (bfloat16 or float16: batch_gemm_softmax.cu:185-197)."""
    D = x.to(dtype)
    m = x.max(dim=-1, keepdim=True).values
    z = torch.exp(x - m).sum(dim=-1, keepdim=True)
    inv = 1.0 / z
    soft = (torch.exp(D.float() - m) * inv).to(dtype)
    return D, m.squeeze(-1), inv.squeeze(-1), soft


def batch_gemm_softmax(q, cent, scale=None):
    """Reference semantics of batch_gemm_softmax: returns (D, norm, inv_sum, softmax)."""
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    return softmax_from_logits(logits_fp32(q, cent, scale), q.dtype)


def dist_from_softmax(soft: torch.Tensor, mask: torch.Tensor = None) -> torch.Tensor:
    """dist = dtype(sum_j float(P_j)) in the element type of the softmax, masked clusters -> finfo(dtype).min
    (cache_hub/retroinfer_cache.py:572-573)."""
    d = soft.float().sum(dim=1).to(soft.dtype)
    if mask is not None:
        d = d.masked_fill(mask.bool(), torch.finfo(soft.dtype).min)
    return d


def select(dist: torch.Tensor, nprobe: int, es: int):
    """Top (nprobe+es) clusters per group, largest first; equal scores are ordered by ascending
    id (torch.topk leaves that order open, retroinfer_cache.py:574).  Returns
    (retrieval ids [BG, nprobe] in rank order, estimation ids [BG, es] ascending)."""
    order = torch.sort(dist.float(), dim=-1, descending=True, stable=True).indices
    ret = order[:, :nprobe].contiguous()
    est = torch.sort(order[:, nprobe:nprobe + es], dim=-1).values.contiguous()
    return ret, est


def retrieval_layout(ret_ids, cluster_size, page, max_pages):
    """Which retrieved clusters fit the execution buffer: stop before the first cluster whose
    pages push the running total over max_pages
    (library/retroinfer/retroinfer_kernels/src/wave_buffer_cpu.cpp:207-216).
    Returns (kept count per group, token offsets [BG, nprobe+1])."""
    BG, nprobe = ret_ids.shape
    kept = torch.zeros(BG, dtype=torch.int64)
    offs = torch.zeros(BG, nprobe + 1, dtype=torch.int64)
    for g in range(BG):
        pages = 0
        tok = 0
        k = 0
        for r in range(nprobe):
            sz = int(cluster_size[g, ret_ids[g, r]])
            pages += (sz + page - 1) // page
            if pages > max_pages:
                break
            offs[g, r] = tok
            tok += sz
            k += 1
        offs[g, k:] = tok
        kept[g] = k
    return kept, offs
