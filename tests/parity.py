"""Helpers shared by the parity tests: stage-wise comparison rules.

Rule for selections (cluster ids): they must equal the oracle's on the same scores except for
clusters whose score lies within one bf16 ulp of the zone boundary score, where either side is
acceptable.  Rule for bf16 quantities computed through exp/sum: at most one bf16 ulp apart.
"""
import numpy as np
import torch

from oracle.numerics import bf16_ulp


def bf16_bits_i(x):
    """int32 view of bf16 bit patterns mapped so that consecutive floats are consecutive ints."""
    b = x.contiguous().view(torch.int16).to(torch.int32) & 0xFFFF
    return torch.where(b >= 0x8000, 0x8000 - b, b)


def ulp_distance_bf16(a, b):
    return (bf16_bits_i(a) - bf16_bits_i(b)).abs()


def check_zone_sets(dist, ret, est, ret_ref, est_ref, nprobe, es, band=1.0):
    """dist [BG, nc] bf16 (oracle or common scores); ret/est: ids under test; *_ref: oracle ids.
    Returns the number of tolerated boundary swaps; asserts on anything else."""
    d = dist.float()
    swaps = 0
    for g in range(d.shape[0]):
        srt = torch.sort(d[g], descending=True, stable=True).values
        for got, ref, rank in ((ret[g], ret_ref[g], nprobe), (est[g], est_ref[g], nprobe + es)):
            if got.numel() == 0:
                continue
            sg, sr = set(got.tolist()), set(ref.tolist())
            assert len(sg) == got.numel(), f"group {g}: duplicate ids in a zone"
            if sg == sr:
                continue
            bounds = [srt[rank - 1]]
            if rank != nprobe:
                bounds.append(srt[nprobe - 1])
            for c in sg ^ sr:
                ok = any(abs(float(d[g, c]) - float(t)) <= band * float(bf16_ulp(t.reshape(1))) for t in bounds)
                assert ok, f"group {g}: cluster {c} score {float(d[g, c])} is not a boundary tie ({[float(t) for t in bounds]})"
                swaps += 1
    return swaps


def check_rank_order(dist, ret, band=1.0):
    """retrieval ids must come in non-increasing score order (within the band)."""
    d = dist.float()
    for g in range(d.shape[0]):
        s = d[g, ret[g].long()]
        viol = s[1:] - s[:-1]
        lim = band * bf16_ulp(s[1:])
        assert bool((viol <= lim).all()), f"group {g}: retrieval zone not in rank order"
