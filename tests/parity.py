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


# label -> [checks, swaps within one ulp, swaps between one ulp and the band]; printed at the end of a run
TIE_TALLY = {}


class ZoneSwaps(int):
    """Number of tolerated boundary swaps; `.beyond1` of them lie further than one bf16 ulp (and at most
    `band` ulps) from the boundary score."""
    beyond1 = 0


def check_zone_sets(dist, ret, est, ret_ref, est_ref, nprobe, es, band=1.0, label=None):
    """dist [BG, nc] bf16 (oracle or common scores); ret/est: ids under test; *_ref: oracle ids.
    Returns the number of tolerated boundary swaps (a ZoneSwaps: .beyond1 counts those whose score is
    more than one ulp from the boundary); asserts on anything else."""
    d = dist.float()
    swaps, beyond1 = 0, 0
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
                ulps = min(abs(float(d[g, c]) - float(t)) / float(bf16_ulp(t.reshape(1))) for t in bounds)
                assert ulps <= band, f"group {g}: cluster {c} score {float(d[g, c])} is not a boundary tie ({[float(t) for t in bounds]})"
                swaps += 1
                beyond1 += ulps > 1.0
    out = ZoneSwaps(swaps)
    out.beyond1 = int(beyond1)
    if label is not None:
        t = TIE_TALLY.setdefault(label, [0, 0, 0])
        t[0] += 1; t[1] += swaps - int(beyond1); t[2] += int(beyond1)
    return out


def check_rank_order(dist, ret, band=1.0):
    """retrieval ids must come in non-increasing score order (within the band)."""
    d = dist.float()
    for g in range(d.shape[0]):
        s = d[g, ret[g].long()]
        viol = s[1:] - s[:-1]
        lim = band * bf16_ulp(s[1:])
        assert bool((viol <= lim).all()), f"group {g}: retrieval zone not in rank order"
