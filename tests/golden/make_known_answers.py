"""Writes tests/golden/known_answers.json: small known-answer cases for the wave-index path.

The reference stores no golden vectors for this path (its two test scripts draw random inputs and
compare with torch), so these cases are worked out from the rules of the reference's code with
integers, exact fractions and hand-listed traces.  Nothing here calls the CPU restatement under
oracle/ or the library: the file is an independent statement of what both must produce.

Run from the repository root:  python tests/golden/make_known_answers.py
"""
import json
import math
import os
import struct
from fractions import Fraction


def f32(x):
    """Nearest float32 of a Python float (exact products and sums of float32 fit a double)."""
    return struct.unpack("f", struct.pack("f", x))[0]


def bf16(x):
    """Nearest-even bfloat16 of a number, as a float."""
    bits = struct.unpack("I", struct.pack("f", f32(float(x))))[0]
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return struct.unpack("f", struct.pack("I", bits))[0]


# ---------------------------------------------------------------------------------------------
# k-means initial token per centroid (cache_hub/kmeans.py:234-237): two float32 roundings, one for
# the product and one for the sum, then truncation.
def init_indices(n_tokens, nc):
    step, half = f32(n_tokens / nc), f32(n_tokens / nc / 2)
    return [int(f32(f32(f32(float(i)) * step) + half)) for i in range(nc)]


INIT_CASES = [(8192, 512), (131072, 8192), (61440, 3840), (262144, 16384), (1000, 7), (1024, 64), (96, 32),
              (100000, 96), (131072 + 37, 8192)]


# ---------------------------------------------------------------------------------------------
# A clustering whose every step can be followed by hand (cache_hub/kmeans.py:224-259).
# 96 tokens, 32 centroids, dimension 128.  Token t = amplitude[t % 3] * e_(t // 3) with amplitudes
# 1, 2, 3, except:
#   token 3            = e_1 + 2 e_2      (scores 2 against centroid 1 = 2 e_1, 4 against centroid 2 = 2 e_2:
#                                          it moves to cluster 2 and stays there)
#   tokens 15, 16, 17  = 1.5 e_5, 0, 4.5 e_5   (centroid 5 starts as token 16 = 0: every score of these three
#                                          tokens is 0, the first index wins the tie, they join cluster 0 and
#                                          cluster 5 stays empty with its centroid unchanged)
# Initial centroid i is token 3 i + 1 (n_tokens / nc = 3 exactly).  After any number of iterations:
#   cluster 0 = {0,1,2,15,16,17}, mean = (6 e_0 + 6 e_5) / 6 = e_0 + e_5
#   cluster 1 = {4,5},            mean = 2.5 e_1
#   cluster 2 = {3,6,7,8},        mean = (e_1 + 8 e_2) / 4 = 0.25 e_1 + 2 e_2
#   cluster 5 = {},               centroid stays 0, masked
#   cluster i = {3i,3i+1,3i+2},   mean = 2 e_i
# (cluster 2's normalised centroid between iterations is (e_1 + 8 e_2)/sqrt(65): token 3 scores
# 17/sqrt(65) = 2.1 there against 1 at centroid 1, so it stays.)  Values: token t carries
# (t % 7 + 1) e_0 + e_127, so value_sum[c] = (sum of t % 7 + 1, cluster size) in those two coordinates.
def kmeans_case():
    n, nc, dim = 96, 32, 128
    keys = []      # sparse rows: {coordinate: value}
    for t in range(n):
        keys.append({t // 3: float((1, 2, 3)[t % 3])})
    keys[3] = {1: 1.0, 2: 2.0}
    keys[15], keys[16], keys[17] = {5: 1.5}, {}, {5: 4.5}
    assign = [t // 3 for t in range(n)]
    assign[3] = 2
    assign[15] = assign[16] = assign[17] = 0
    clusters = [[t for t in range(n) if assign[t] == c] for c in range(nc)]
    cent = []
    for c in range(nc):
        if not clusters[c]:
            cent.append({})        # the zero token it started from
            continue
        acc = {}
        for t in clusters[c]:
            for k, v in keys[t].items():
                acc[k] = acc.get(k, Fraction(0)) + Fraction(v)
        cent.append({k: bf16(float(v / len(clusters[c]))) for k, v in acc.items() if v != 0})
    vsum = []
    for c in range(nc):
        s = sum(t % 7 + 1 for t in clusters[c])
        assert s < 256                      # exact in bfloat16
        vsum.append({0: float(s), 127: float(len(clusters[c]))} if clusters[c] else {})
    assert cent[0] == {0: 1.0, 5: 1.0} and cent[1] == {1: 2.5} and cent[2] == {1: 0.25, 2: 2.0}
    return dict(n_tokens=n, n_centroids=nc, dim=dim,
                keys=[{str(k): v for k, v in r.items()} for r in keys],
                values=[{"0": float(t % 7 + 1), "127": 1.0} for t in range(n)],
                init=[3 * i + 1 for i in range(nc)], assign=assign, clusters=clusters,
                cluster_size=[len(c) for c in clusters],
                centroids=[{str(k): v for k, v in r.items()} for r in cent],
                value_sum=[{str(k): v for k, v in r.items()} for r in vsum])


# ---------------------------------------------------------------------------------------------
# Scoring (batch_gemm_softmax.cu:171-198, retroinfer_cache.py:572-575) where the softmax is known in closed form.
_X = f32(512.0 * f32(1.0 / math.sqrt(128.0)))
DOMINANT = bf16(math.exp(bf16(_X) - _X))
assert bf16(_X) == 45.25 and DOMINANT == 0.99609375 and bf16(4 * DOMINANT) == 3.984375


def scoring_cases():
    return [
        # 8 identical centroids: every head's softmax is 1/8, the score sum over 4 heads is 0.5
        dict(name="uniform", gs=4, nc=8, q_coord=0, q_amp=3.0, cent=[{"0": 1.0}] * 8,
             softmax=[[0.125] * 8] * 4, dist=[0.5] * 8),
        # one centroid ahead by a logit gap of 45: nothing else contributes to the sum (below 1e-19), so
        # its softmax would be 1 -- but the final value is computed from the logit rounded to bfloat16
        # against the float32 row maximum (batch_gemm_softmax.h:237-239): x = 512/sqrt(128) = 45.2548...,
        # bf16(x) = 45.25, value = bf16(exp(45.25 - x)) = 0.99609375; score sum over 4 heads = 3.984375
        dict(name="dominant", gs=4, nc=8, q_coord=0, q_amp=64.0,
             cent=[{}, {}, {}, {"0": 8.0}, {}, {}, {}, {}],
             softmax=[[0.0, 0.0, 0.0, DOMINANT, 0.0, 0.0, 0.0, 0.0]] * 4,
             dist=[0.0, 0.0, 0.0, bf16(4 * DOMINANT), 0.0, 0.0, 0.0, 0.0]),
    ]


# Selection (retroinfer_cache.py:573-575): largest scores first, masked clusters last, equal scores by
# ascending id; first nprobe = retrieval zone in rank order, next es = estimation zone (any order:
# compared as a set).  Scores given directly as centroids along the query so the score order is known:
# centroid amplitude a gives logit a * q_amp / sqrt(128), monotone in a.
def selection_case():
    amps = [2.0, 1.0, 2.0, 3.0, 1.0, 0.5, 2.0, 0.25]      # cluster 3 has the best score but is empty (masked)
    sizes = [9, 8, 0, 0, 17, 1, 4, 3]                      # cluster 2 is empty too: masked
    # unmasked order: 0 (2.0), 6 (2.0), 1 (1.0), 4 (1.0), 5 (0.5), 7 (0.25); then masked 2, 3
    return dict(gs=4, nc=8, q_amp=16.0, amps=amps, sizes=sizes, nprobe=3, es=2,
                ret=[0, 6, 1], est=[4, 5])


# Execution-buffer cut-off (wave_buffer_cpu.cpp:207-216): stop before the first cluster whose pages
# push the running total over max_pages.  sizes 17, 0, 9, 1, 8 in rank order, 8 tokens per page, 5 pages:
# 3 pages -> 3, +0 -> 3, +2 -> 5 (fits), +1 -> 6 (stop).  Three ranks kept, 26 tokens.
def layout_case():
    return dict(cluster_size=[9, 8, 0, 17, 1], ret=[3, 2, 0, 4, 1], page=8, max_pages=5,
                kept=3, token_offsets=[0, 17, 17, 26], tokens=26)


# ---------------------------------------------------------------------------------------------
# Block cache trace (wave_buffer_cpu.cpp:190-257 access, :102-188 update), followed by hand.
# 8 tokens per block, 4 cache blocks, 6 buffer blocks.  Cluster sizes 8, 16, 5, 0, 20, 8 tokens
# (1, 2, 1, 0, 3, 1 blocks), first store rows 0, 8, 24, 29, 29, 49.  Free block ids are handed out
# 0, 1, 2, ... and a released cluster's ids are reused last-released-first (the reference's come from an
# unordered_set, wave_buffer_cpu.cpp:153-156: which id a block gets is the library's choice).
# Entries: hits (cache block, tokens, token offset among hits); misses (store row, tokens, token offset
# among misses); updates (cache block, tokens, token offset in the miss part of the buffer).
def lru_trace():
    return dict(
        block=8, capacity=4, buffer_size=6, sizes=[8, 16, 5, 0, 20, 8],
        steps=[
            # (every step probes four ids: the empty cluster 3 fills up the shorter ones)
            # cold: cluster 1 (2 blocks) and 0 miss, the empty cluster 3 is skipped; both admitted
            dict(ids=[1, 3, 0, 3], hit=[], miss=[[8, 8, 0], [16, 8, 8], [0, 8, 16]],
                 update=[[0, 8, 0], [1, 8, 8], [2, 8, 16]], resident={"1": [0, 1], "0": [2]}),
            # 0 hits; 4 (3 blocks) and 2 (1 block) miss and need all 4 blocks: 1 and then 0 (the tail
            # after the touch) are evicted, 4 takes the ids released last
            dict(ids=[0, 4, 2, 3], hit=[[2, 8, 0]], miss=[[29, 8, 0], [37, 8, 8], [45, 4, 16], [24, 5, 20]],
                 update=[[2, 8, 0], [0, 8, 8], [1, 4, 16], [3, 5, 20]], resident={"4": [2, 0, 1], "2": [3]}),
            # 1 misses (2 blocks), 2 hits, 5 misses, 4 would need blocks 5..7 of 6: cut off there.
            # 1 and 5 need 3 blocks: 4 is the least recently used and goes
            dict(ids=[1, 2, 5, 4], hit=[[3, 5, 0]], miss=[[8, 8, 0], [16, 8, 8], [49, 8, 16]],
                 update=[[2, 8, 0], [0, 8, 8], [1, 8, 16]], resident={"2": [3], "1": [2, 0], "5": [1]}),
        ])


# ---------------------------------------------------------------------------------------------
# Weighted attention (call sites retroinfer_cache.py:611-617, 666-674) where the result is rational.
# All keys orthogonal to the query: every logit is 0, exp = 1.
def attention_cases():
    return [
        # estimation call: three clusters of sizes 1, 2, 5 with value sums 8 e_0, 16 e_1, 40 e_2:
        # out = (sum of value sums) / (sum of sizes) = e_0 + 2 e_1 + 5 e_2, lse = log 8
        dict(name="weighted_zero_logits", weights=[1.0, 2.0, 5.0],
             values=[{"0": 8.0}, {"1": 16.0}, {"2": 40.0}], out={"0": 1.0, "1": 2.0, "2": 5.0}, lse=math.log(8.0)),
        # final call: 8 tokens with values 4 e_3 merged into a previous partial result (out 2 e_0 at
        # lse log 8): equal masses, out = (2 e_0 + 4 e_3) / 2 = e_0 + 2 e_3, lse = log 16
        dict(name="merge_equal_mass", weights=None, values=[{"3": 4.0}] * 8, previous_out={"0": 2.0},
             previous_lse=math.log(8.0), out={"0": 1.0, "3": 2.0}, lse=math.log(16.0)),
    ]


def main():
    out = dict(
        init_indices=[dict(n_tokens=n, n_centroids=c, first=init_indices(n, c)[:4], last=init_indices(n, c)[-2:],
                           sum=sum(init_indices(n, c))) for n, c in INIT_CASES],
        kmeans=kmeans_case(), scoring=scoring_cases(), selection=selection_case(), layout=layout_case(),
        lru=lru_trace(), attention=attention_cases())
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "known_answers.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    print("wrote", path)


if __name__ == "__main__":
    main()
