"""Seeded synthetic KV for parity tests and the benchmark, plus the derivation of the index
parameters from a context length (benchmark/config.py:17-56 of the reference)."""
import math

import torch

STEADY_START, STEADY_END = 4, 64


def derive_config(context_len, budget_ratio=0.018, estimate_ratio=0.232, n_segments=None, n_clusters=None):
    """n_centroids / n_segment / nprobe / estimation size as benchmark/config.py:26-53 computes
    them (nprobe and the estimation zone are fractions of the cluster count)."""
    if n_segments is None:
        n_segments = max(1, context_len // 8192)
    if n_clusters is None:
        n_clusters = math.ceil(context_len / 16)
        lower = (n_clusters // (n_segments * 32)) * (n_segments * 32)
        upper = lower + n_segments * 32
        n_clusters = lower if abs(n_clusters - lower) <= abs(n_clusters - upper) else upper
    nprobe = max(1, int(n_clusters * budget_ratio))
    es = int(n_clusters * estimate_ratio)
    return {
        "n_centroids": n_clusters, "n_segment": n_segments, "nprobe": nprobe,
        "cache_cluster_num": 3 * nprobe, "max_compute_cluster_num": es + nprobe,
        "static_pattern_start": STEADY_START, "static_pattern_end": STEADY_END, "cache_unit_size": 8,
    }


def group_seed(seed, b, h):
    return seed * 1_000_003 + b * 1009 + h


def make_group(seed, b, h, n_tokens, n_centers, gs, dim=128, outliers=False, sigma=0.3, n_extra=0,
               device="cpu"):
    """One (sequence, kv head): keys from a Gaussian mixture (N(0,1) centres, per-token noise
    sigma, optionally 4 outlier channels scaled x8), N(0,1) values and queries.  Returns fp32
    (keys [n_tokens + n_extra, dim], values, q [gs, dim]); the extra tokens serve as steady zone."""
    g = torch.Generator(device=device).manual_seed(group_seed(seed, b, h))
    kw = dict(generator=g, device=device, dtype=torch.float32)
    centers = torch.randn(n_centers, dim, **kw)
    n = n_tokens + n_extra
    if outliers:
        ch = torch.randperm(dim, generator=g, device=device)[:4]
        centers[:, ch] *= 8
    assign = torch.randint(n_centers, (n,), generator=g, device=device)
    noise = sigma * torch.randn(n, dim, **kw)
    if outliers:
        noise[:, ch] *= 8
    keys = centers[assign] + noise
    values = torch.randn(n, dim, **kw)
    q = torch.randn(gs, dim, **kw)
    return keys, values, q


def make_batch(seed, batch, kv_heads, n_tokens, n_centers, gs, dim=128, outliers=False, n_extra=0,
               device="cpu", dtype=torch.bfloat16):
    """Stacks make_group over (batch, kv head): keys/values [B, Hkv, n, dim], q [B, Hkv*gs, dim]."""
    ks, vs, qs = [], [], []
    for b in range(batch):
        kb, vb, qb = [], [], []
        for h in range(kv_heads):
            k, v, q = make_group(seed, b, h, n_tokens, n_centers, gs, dim, outliers, n_extra=n_extra, device=device)
            kb.append(k.to(dtype)); vb.append(v.to(dtype)); qb.append(q.to(dtype))
        ks.append(torch.stack(kb)); vs.append(torch.stack(vb)); qs.append(torch.cat(qb))
    return torch.stack(ks), torch.stack(vs), torch.stack(qs)
