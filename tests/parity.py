"""Helpers shared by the parity tests: stage-wise comparison rules.

Rule for selections (cluster ids): they must equal the oracle's on the same scores except for
clusters whose score lies within one bf16 ulp of the zone boundary score, where either side is
acceptable.  Rule for bf16 quantities computed through exp/sum: at most one bf16 ulp apart.
Rule for cluster scores (a bf16 sum of bf16-rounded probabilities): inside the interval `score_interval`
gives, i.e. each head's probability may round either way only where the fp32 exp/normaliser tolerance
reaches a bf16 rounding boundary; one such flip of the dominant head plus the final rounding is two ulps.

End to end (kernel selections against the oracle's OWN logits) one more thing is legitimate: the score
pipeline rounds every logit to bf16 first, and two fp32 accumulation orders of the same dot product can
land on different sides of a bf16 rounding boundary.  Such a flip moves that head's probability by a bf16
ulp of the LOGIT (up to e^(2^-8 |x|) - 1, a few percent), i.e. the cluster's score by several of its own
ulps.  `flip_slack` bounds that per cluster from the logits' own tolerance, and the end-to-end checks add
it to the band; the tally reports how often it was needed.
"""
import numpy as np
import torch

from oracle.numerics import bf16_ulp, ulp16


def bf16_bits_i(x):
    """int32 view of bf16 bit patterns mapped so that consecutive floats are consecutive ints."""
    b = x.contiguous().view(torch.int16).to(torch.int32) & 0xFFFF
    return torch.where(b >= 0x8000, 0x8000 - b, b)


def ulp_distance_bf16(a, b):
    return (bf16_bits_i(a) - bf16_bits_i(b)).abs()


def score_interval(logits, mask=None, rel=4e-6, dtype=torch.bfloat16):
    """(lo, hi) bf16 [BG, nc]: the scores bf16(sum_j bf16(p_j)) with every head's probability
    p_j = exp(bf16(x_j) - m_j) / Z_j (evaluated in float64 from fp32 logits [BG, gs, nc]) scaled by
    (1 - rel) and (1 + rel), the bf16 probabilities added in fp32 in head order.  rel covers a fast fp32 exp, the order of the fp32 sum behind Z and a
    reciprocal instead of a division (each around 1e-7 .. 1e-6 relative).  Both roundings are monotone,
    so any implementation within that tolerance lands in [lo, hi]; lo == hi for all but the few clusters
    with a head sitting on a rounding boundary."""
    x = logits.double()
    m = x.max(dim=-1, keepdim=True).values
    z = torch.exp(x - m).sum(dim=-1, keepdim=True)
    p = torch.exp(logits.to(dtype).double() - m) / z
    out = []
    for f in (1.0 - rel, 1.0 + rel):
        pb = (p * f).float().to(dtype).float()
        d = torch.zeros_like(pb[:, 0])
        for j in range(pb.shape[1]):   # fp32 sum in head order: a head of 2^-24 of the sum can decide a tie
            d = d + pb[:, j]
        d = d.to(dtype)
        if mask is not None:
            d = d.masked_fill(mask.bool(), torch.finfo(dtype).min)
        out.append(d)
    return out[0], out[1]


# label -> [checks, swaps within one ulp, swaps between one ulp and the band]; printed at the end of a run
TIE_TALLY = {}
# label -> decisions that were only acceptable because of a logit's bf16 rounding flip
FLIP_TALLY = {}


def flip_slack(logits, dist_of, delta=2e-5):
    """Per-cluster score uncertainty [BG, nc] (float) caused by logits within `delta` (the tolerance of the
    fp32 logits) of a bf16 rounding boundary: the scores are recomputed with every logit moved up and down by
    delta (a uniform shift leaves the softmax itself unchanged, so only flipped roundings show), and the two
    deviations are added.  dist_of(logits) -> bf16 scores [BG, nc]."""
    d0 = dist_of(logits).float()
    return (dist_of(logits + delta).float() - d0).abs() + (dist_of(logits - delta).float() - d0).abs()


class ZoneSwaps(int):
    """Number of tolerated boundary swaps; `.beyond1` of them lie further than one bf16 ulp (and at most
    `band` ulps) from the boundary score."""
    beyond1 = 0


def check_zone_sets(dist, ret, est, ret_ref, est_ref, nprobe, es, band=1.0, label=None, slack=None):
    """dist [BG, nc] bf16 (oracle or common scores); ret/est: ids under test; *_ref: oracle ids.
    Returns the number of tolerated boundary swaps (a ZoneSwaps: .beyond1 counts those whose score is
    more than one ulp from the boundary); asserts on anything else.  slack [BG, nc] (optional): per-cluster
    score uncertainty from flip_slack, added for the cluster and for the worst cluster it can swap with."""
    ulp = lambda t: ulp16(t, dist.dtype if dist.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16)
    d = dist.float()
    swaps, beyond1, flips = 0, 0, 0
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
            diff = sorted(sg ^ sr)
            worst = max(float(slack[g, c]) for c in diff) if slack is not None else 0.0
            for c in diff:
                extra = (float(slack[g, c]) + worst) if slack is not None else 0.0
                ulps = min(abs(float(d[g, c]) - float(t)) / float(ulp(t.reshape(1))) for t in bounds)
                flip = min((abs(float(d[g, c]) - float(t)) - extra) / float(ulp(t.reshape(1))) for t in bounds)
                assert flip <= band, f"group {g}: cluster {c} score {float(d[g, c])} is not a boundary tie ({[float(t) for t in bounds]})"
                if ulps > band:          # acceptable only because of a rounding flip of a logit
                    flips += 1
                    continue
                swaps += 1
                beyond1 += ulps > 1.0
    out = ZoneSwaps(swaps)
    out.beyond1 = int(beyond1)
    if label is not None:
        t = TIE_TALLY.setdefault(label, [0, 0, 0])
        t[0] += 1; t[1] += swaps - int(beyond1); t[2] += int(beyond1)
        if flips:
            FLIP_TALLY[label] = FLIP_TALLY.get(label, 0) + flips
    return out


def check_rank_order(dist, ret, band=1.0, slack=None, label=None):
    """retrieval ids must come in non-increasing score order (within the band; with slack [BG, nc] from
    flip_slack, within the band plus the uncertainty of the two neighbours)."""
    d = dist.float()
    for g in range(d.shape[0]):
        ids = ret[g].long()
        s = d[g, ids]
        viol = s[1:] - s[:-1]
        lim = band * ulp16(s[1:], dist.dtype if dist.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16)
        if slack is not None:
            sl = slack[g, ids]
            flips = int(((viol > lim) & (viol <= lim + sl[1:] + sl[:-1])).sum())
            if flips and label is not None:
                FLIP_TALLY[label] = FLIP_TALLY.get(label, 0) + flips
            lim = lim + sl[1:] + sl[:-1]
        assert bool((viol <= lim).all()), f"group {g}: retrieval zone not in rank order"


class BlockIdMap:
    """Bijection between the cache block ids of two block cache managers that follow the same policy but hand
    out free ids in different orders: ids are bound when a cluster is admitted, must translate consistently
    while the cluster is resident, and are forgotten when it is evicted (`retain` keeps the reference ids that
    are still in use)."""

    def __init__(self):
        self.fwd, self.back = {}, {}

    def bind(self, got, ref):
        assert got not in self.fwd and ref not in self.back, "block id handed out twice"
        self.fwd[got], self.back[ref] = ref, got

    def to_ref(self, got):
        return self.fwd[got]

    def retain(self, live_ref_ids):
        for ref in [r for r in self.back if r not in live_ref_ids]:
            del self.fwd[self.back.pop(ref)]
