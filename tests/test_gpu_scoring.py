"""Scoring and selection kernels against the oracle (GPU)."""
import math

import pytest
import torch

from oracle import scoring
from oracle.numerics import bf16_ulp
from tests.parity import (bf16_bits_i, check_zone_sets, check_rank_order, flip_slack, score_interval,
                          ulp_distance_bf16)

pytestmark = pytest.mark.gpu


def _mixture(BG, gs, nc, seed, outliers=True, dt=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    cent = torch.randn(BG, nc, 128, generator=g)
    if outliers:
        cent[:, :, :4] *= 8
    q = torch.randn(BG, gs, 128, generator=g)
    return q.to(dt), cent.to(dt)


def test_batch_gemm_softmax_matches_reference_test(dev):
    """Shape and tolerance of library/retroinfer/test/test_batch_gemm_softmax.py (atol 1e-3),
    with 16 groups instead of 128 to keep the CPU side short."""
    from retrievalattention_amd import kernels
    BG, gs, n, d = 16, 4, 8200, 128
    g = torch.Generator().manual_seed(0)
    q = torch.randn(BG, gs, d, generator=g).to(torch.bfloat16)
    c = torch.randn(BG, n, d, generator=g).to(torch.bfloat16)
    nt = (n + 255) // 256
    D = torch.zeros(BG, gs, n, dtype=torch.bfloat16, device=dev)
    S = torch.zeros_like(D)
    norm = torch.zeros(BG, gs, nt, dtype=torch.float32, device=dev)
    ssum = torch.zeros_like(norm)
    kernels.batch_gemm_softmax(q.to(dev), c.to(dev), D, norm, ssum, S, BG, gs, n, d, 1 / math.sqrt(d), 0)
    torch.cuda.synchronize()
    # the reference's oracle: bmm / sqrt(d) -> softmax, in bf16 tensors
    ref = torch.softmax((torch.bmm(q.float(), c.float().transpose(1, 2)) / math.sqrt(d)), dim=-1)
    assert torch.allclose(S.cpu().float(), ref, atol=1e-3)
    # stage-wise: D is the bf16 rounding of the fp32 logits up to accumulation order
    Dr, m, inv, Sr = scoring.batch_gemm_softmax(q, c)
    dd = ulp_distance_bf16(D.cpu(), Dr)
    near_zero = (D.cpu().float() - Dr.float()).abs() <= 1e-5   # ulps mean nothing next to 0
    assert bool(((dd <= 1) | near_zero).all())
    assert float((dd > 0).float().mean()) < 2e-3
    # final row max / inverse sum sit in slot 0 of Norm / Sum
    fm = norm.view(BG, -1)[:, :gs].cpu()
    fi = ssum.view(BG, -1)[:, :gs].cpu()
    assert torch.allclose(fm, m, rtol=0, atol=1e-5)
    assert torch.allclose(fi, inv, rtol=1e-5)
    # softmax given the kernel's own D and statistics: at most one bf16 ulp from the oracle's formula
    Sg = (torch.exp(D.cpu().float() - fm[..., None]) * fi[..., None]).to(torch.bfloat16)
    assert int(ulp_distance_bf16(S.cpu(), Sg).max()) <= 1


def test_batch_gemm_softmax_half(dev):
    """The operator on IEEE half tensors (batch_gemm_softmax.cu:185-197 accepts Half): the reference's test
    oracle and tolerance (test_batch_gemm_softmax.py: bmm / sqrt(d) -> softmax, atol 1e-3), and stage by
    stage: D is the fp16 rounding of the fp32 logits up to accumulation order, the statistics come from the
    fp32 logits, the softmax from the kernel's own D within one fp16 ulp."""
    from retrievalattention_amd import kernels
    BG, gs, n, d = 6, 5, 4104, 128
    g = torch.Generator().manual_seed(1)
    q = torch.randn(BG, gs, d, generator=g).to(torch.float16)
    c = torch.randn(BG, n, d, generator=g).to(torch.float16)
    nt = (n + 255) // 256
    D = torch.zeros(BG, gs, n, dtype=torch.float16, device=dev)
    S = torch.zeros_like(D)
    norm = torch.zeros(BG, gs, nt, dtype=torch.float32, device=dev)
    ssum = torch.zeros_like(norm)
    kernels.batch_gemm_softmax(q.to(dev), c.to(dev), D, norm, ssum, S, BG, gs, n, d, 1 / math.sqrt(d), 0)
    torch.cuda.synchronize()
    logits = torch.bmm(q.double(), c.double().transpose(1, 2)) / math.sqrt(d)
    ref = torch.softmax(logits, dim=-1)
    assert torch.allclose(S.cpu().double(), ref, atol=1e-3)
    # D: fp16(fp32 logits); an fp16 ulp at |x| is 2^-10 |x| (2^-24 below the normal range)
    err = (D.cpu().double() - logits).abs()
    assert bool((err <= logits.abs() * 2.0 ** -10 + 2.0 ** -24 + 1e-5).all())
    fm = norm.view(BG, -1)[:, :gs].cpu().double()
    fi = ssum.view(BG, -1)[:, :gs].cpu().double()
    assert torch.allclose(fm, logits.max(dim=-1).values, rtol=0, atol=1e-5)
    assert torch.allclose(fi, 1.0 / torch.exp(logits - logits.max(dim=-1, keepdim=True).values).sum(-1), rtol=1e-5)
    Sg = torch.exp(D.cpu().double() - fm[..., None]) * fi[..., None]
    assert bool(((S.cpu().double() - Sg).abs() <= Sg * 2.0 ** -10 + 2.0 ** -24).all())
    # mixing element types is refused
    with pytest.raises(TypeError):
        kernels.batch_gemm_softmax(q.to(dev), c.to(dev).to(torch.bfloat16), D, norm, ssum, S, BG, gs, n, d, 1.0, 0)


@pytest.mark.parametrize("BG,gs,nc,nprobe,es,seed", [
    (8, 4, 512, 9, 118, 0),       # config-1 shape
    (4, 4, 8192, 147, 1900, 1),   # config-2 shape, fewer groups
    (4, 7, 3840, 69, 890, 2),     # config-4 shape (gs = 7)
    (2, 8, 16384, 294, 3801, 3),  # config-5 shape
    (3, 1, 64, 1, 0, 4),          # smallest: one probe, no estimation zone
    (2, 16, 1000, 20, 980, 5),    # nc not a multiple of 256, zones cover every cluster
    (1, 4, 32768, 300, 3000, 6),  # more clusters than the select kernel stages in LDS
    (1, 16, 65536, 1023, 20000, 7),  # 65536 clusters (the most the entry point takes), 16 heads
    (2, 4, 15000, 1500, 2250, 8),    # probe lists of the reference's throughput harness (throughput_eval/test.py:74,
    (1, 4, 30000, 3000, 4500, 9),    #   nprobe = 10 % of the clusters): 240K and 480K tokens of context
    (1, 8, 40960, 4096, 100, 10),    # the longest probe list the entry point takes
    (4096, 1, 64, 4, 20, 11),        # as many groups as an attention launch takes
])
def test_score_select(dev, BG, gs, nc, nprobe, es, seed, dt=torch.bfloat16):
    from retrievalattention_amd import kernels
    q, cent = _mixture(BG, gs, nc, seed, dt=dt)
    g = torch.Generator().manual_seed(seed + 100)
    mask = torch.rand(BG, nc, generator=g) < 0.02
    size = torch.randint(1, 40, (BG, nc), generator=g, dtype=torch.int32)
    size[mask] = 0
    start = (torch.cumsum(size, 1) - size).to(torch.int32)
    scale = 1 / math.sqrt(128)
    page, max_pages = 8, max(4 * nprobe, 16) * 2
    k2 = nprobe + es
    o = dict(
        logits=torch.empty(BG, gs, nc, dtype=torch.float32, device=dev),
        dist=torch.empty(BG, nc, dtype=dt, device=dev),
        cI=torch.empty(BG, k2, dtype=torch.int64, device=dev),
        ret=torch.empty(BG, nprobe, dtype=torch.int32, device=dev),
        est=torch.empty(BG, max(es, 1), dtype=torch.int32, device=dev),
        off=torch.empty(BG, nprobe + 1, dtype=torch.int32, device=dev),
        rows=torch.full((BG, max_pages * page), -1, dtype=torch.int32, device=dev),
        meta=torch.empty(BG, 4, dtype=torch.int32, device=dev),
    )
    kernels.score_select(q.to(dev), cent.to(dev), mask.to(torch.uint8).to(dev), size.to(dev), start.to(dev),
                         o["logits"], o["dist"], o["cI"], o["ret"], o["est"] if es else None, o["off"], o["rows"],
                         o["meta"], nprobe, es, page, max_pages, scale)
    torch.cuda.synchronize()
    o = {k: v.cpu() for k, v in o.items()}
    ret, est = o["ret"].long(), o["est"][:, :es].long()

    # (1) logits: fp32 accumulation of exact products, any order
    x_ref = scoring.logits_fp32(q, cent, scale)
    assert torch.allclose(o["logits"], x_ref, rtol=2e-5, atol=2e-5)

    # (2) score pipeline on the kernel's own logits: inside the interval that a 4e-6 relative tolerance of the
    # fp32 probabilities leaves open (the oracle's own value wherever no head sits on a bf16 rounding boundary)
    _, _, _, soft = scoring.softmax_from_logits(o["logits"], dt)
    dist_ref = scoring.dist_from_softmax(soft, mask)
    dd = ulp_distance_bf16(o["dist"], dist_ref)
    lo, hi = score_interval(o["logits"], mask, dtype=dt)
    kb = bf16_bits_i(o["dist"])
    assert bool(((kb >= bf16_bits_i(lo)) & (kb <= bf16_bits_i(hi))).all())
    assert int(ulp_distance_bf16(lo, hi).max()) <= 2 and int(dd.max()) <= 2
    assert float((dd > 0).float().mean()) < 0.02

    # (3) selection is exact on the kernel's own scores (ties by ascending id)
    ret_x, est_x = scoring.select(o["dist"], nprobe, es)
    assert torch.equal(ret, ret_x)
    assert torch.equal(est, est_x)
    assert torch.equal(o["cI"][:, :nprobe], ret_x) and torch.equal(o["cI"][:, nprobe:], est_x)

    # (4) end to end against the oracle's scores: identical up to boundary ties
    dist_of = lambda x: scoring.dist_from_softmax(scoring.softmax_from_logits(x, dt)[3], mask)
    dist_o = dist_of(x_ref)
    ret_o, est_o = scoring.select(dist_o, nprobe, es)
    # the band, plus what a bf16 rounding flip of a logit inside the logits' own tolerance can move a score
    slack = flip_slack(x_ref, dist_of, delta=2e-5)
    label = f"score_select BG{BG} gs{gs} nc{nc}" + (" f16" if dt == torch.float16 else "")
    check_zone_sets(dist_o, ret, est, ret_o, est_o, nprobe, es, band=1.0, label=label, slack=slack)
    check_rank_order(dist_o, ret, band=1.0, slack=slack, label=label)

    # (5) token layout of the retrieved clusters
    kept, offs = scoring.retrieval_layout(ret, size, page, max_pages)
    assert torch.equal(o["meta"][:, 0].long(), kept)
    assert torch.equal(o["off"].long(), offs)
    assert torch.equal(o["meta"][:, 1].long(), offs[:, -1])
    for gi in range(BG):
        exp_rows = torch.cat([start[gi, c] + torch.arange(int(size[gi, c])) for c in ret[gi, :int(kept[gi])]]
                             + [torch.zeros(0, dtype=torch.int64)])
        assert torch.equal(o["rows"][gi, :exp_rows.numel()].long(), exp_rows.long())


@pytest.mark.parametrize("BG,gs,nc,nprobe,es,seed", [
    (8, 4, 512, 9, 118, 20), (4, 4, 8192, 147, 1900, 21), (4, 7, 3840, 69, 890, 22), (2, 8, 16384, 294, 3801, 23),
    (3, 1, 64, 1, 0, 24), (2, 16, 1000, 20, 980, 25), (1, 4, 32768, 300, 3000, 26), (2, 4, 15000, 1500, 2250, 27),
])
def test_score_select_float16(dev, BG, gs, nc, nprobe, es, seed):
    """The same checks with IEEE half elements (the reference's harnesses default to fp16:
    simple_test.py:29, throughput_eval/test.py:28): logits, probabilities and scores round to fp16."""
    test_score_select(dev, BG, gs, nc, nprobe, es, seed, dt=torch.float16)


def test_score_select_many_seeds(dev):
    """The benchmark shape's selection over 24 more seeds: every check of test_score_select, so the tally
    printed at the end of the run counts how often a zone boundary is decided by a tie inside the one-ulp band
    (and that none needs more)."""
    for seed in range(200, 224):
        test_score_select(dev, 4, 4, 8192, 147, 1900, seed)


def test_score_select_random_shapes(dev):
    """Every check of test_score_select over 60 shapes drawn from a fixed seed: 1..5 groups, group sizes 1..16
    (not only the powers of two the models use), 32..48000 clusters in steps of 8, any retrieval zone up to
    1023 clusters and any estimation zone, including none; then 8 shapes with 1024..4096 probes."""
    import random
    rnd = random.Random(777)
    for it in range(60):
        BG = rnd.choice([1, 2, 3, 5])
        gs = rnd.choice([1, 2, 3, 4, 5, 7, 8, 9, 12, 16])
        nc = 8 * rnd.randint(4, rnd.choice([64, 600, 3000, 6000]))
        nprobe = rnd.randint(1, min(1023, max(1, nc // 4)))
        es = 0 if rnd.random() < 0.2 else rnd.randint(0, nc - nprobe)
        test_score_select(dev, BG, gs, nc, nprobe, es, 1000 + it)
    for it in range(8):   # probe lists past 1023 (several ranks per thread in the layout phase)
        BG, gs = rnd.choice([1, 2]), rnd.choice([1, 4, 7, 8, 16])
        nc = 8 * rnd.randint(640, 5000)
        nprobe = rnd.randint(1024, min(4096, nc // 3))
        es = rnd.randint(0, nc - nprobe)
        test_score_select(dev, BG, gs, nc, nprobe, es, 1100 + it)


def test_score_select_random_shapes_float16(dev):
    """Twenty of the random shapes with IEEE half elements, four of them with more than 1023 probes."""
    import random
    rnd = random.Random(778)
    for it in range(20):
        BG = rnd.choice([1, 2, 3])
        gs = rnd.choice([1, 2, 3, 4, 5, 7, 8, 9, 12, 16])
        if it < 16:
            nc = 8 * rnd.randint(4, rnd.choice([64, 600, 3000, 6000]))
            nprobe = rnd.randint(1, min(1023, max(1, nc // 4)))
        else:
            nc = 8 * rnd.randint(640, 4000)
            nprobe = rnd.randint(1024, min(4096, nc // 3))
        es = 0 if rnd.random() < 0.2 else rnd.randint(0, nc - nprobe)
        test_score_select(dev, BG, gs, nc, nprobe, es, 1200 + it, dt=torch.float16)


@pytest.mark.parametrize("kind", ["all_equal", "mostly_masked", "two_values"])
def test_score_select_degenerate_scores(dev, kind):
    """Score distributions that put (nearly) every cluster on one score: identical centroids, 97 % of the
    clusters masked as empty, two distinct scores.  The zones are then decided by the id order of ties alone and
    must equal the oracle's selection on the kernel's own scores exactly."""
    from retrievalattention_amd import kernels
    BG, gs, nc, nprobe, es = 3, 4, 2048, 37, 480
    g = torch.Generator().manual_seed(11)
    q = torch.randn(BG, gs, 128, generator=g).to(torch.bfloat16)
    base = torch.randn(BG, 1, 128, generator=g)
    cent = base.expand(BG, nc, 128).clone()
    mask = torch.zeros(BG, nc, dtype=torch.bool)
    if kind == "mostly_masked":
        cent = torch.randn(BG, nc, 128, generator=g)
        mask = torch.rand(BG, nc, generator=g) < 0.97
        mask[:, :nprobe + es + 5] = False          # enough live clusters for both zones, at the low ids
    elif kind == "two_values":
        cent[:, ::3] = -cent[:, ::3]
    cent = cent.to(torch.bfloat16)
    size = torch.randint(1, 20, (BG, nc), generator=g, dtype=torch.int32)
    size[mask] = 0
    start = (torch.cumsum(size, 1) - size).to(torch.int32)
    k2 = nprobe + es
    logits = torch.empty(BG, gs, nc, dtype=torch.float32, device=dev)
    dist = torch.empty(BG, nc, dtype=torch.bfloat16, device=dev)
    cI = torch.empty(BG, k2, dtype=torch.int64, device=dev)
    ret = torch.empty(BG, nprobe, dtype=torch.int32, device=dev)
    est = torch.empty(BG, es, dtype=torch.int32, device=dev)
    off = torch.empty(BG, nprobe + 1, dtype=torch.int32, device=dev)
    meta = torch.empty(BG, 4, dtype=torch.int32, device=dev)
    kernels.score_select(q.to(dev), cent.to(dev), mask.to(torch.uint8).to(dev), size.to(dev), start.to(dev), logits,
                         dist, cI, ret, est, off, None, meta, nprobe, es, 8, 4096, 1 / math.sqrt(128))
    torch.cuda.synchronize()
    ret_x, est_x = scoring.select(dist.cpu(), nprobe, es)
    assert torch.equal(ret.cpu().long(), ret_x) and torch.equal(est.cpu().long(), est_x)
    if kind == "all_equal":      # every score the same: the zones are the lowest ids
        assert torch.equal(ret_x, torch.arange(nprobe).expand(BG, nprobe))
        assert torch.equal(est_x, torch.arange(nprobe, k2).expand(BG, es))
    kept, offs = scoring.retrieval_layout(ret.cpu().long(), size, 8, 4096)
    assert torch.equal(meta.cpu()[:, 0].long(), kept) and torch.equal(off.cpu().long(), offs)


def test_score_select_page_cutoff(dev):
    """A tiny execution buffer forces the reference's cut-off: clusters after the first one that
    does not fit are dropped (wave_buffer_cpu.cpp:207-216)."""
    from retrievalattention_amd import kernels
    BG, gs, nc, nprobe, es = 2, 4, 256, 16, 32
    q, cent = _mixture(BG, gs, nc, 7)
    size = torch.full((BG, nc), 20, dtype=torch.int32)
    start = (torch.cumsum(size, 1) - size).to(torch.int32)
    page, max_pages = 8, 10  # 3 pages per cluster -> only 3 clusters fit
    logits = torch.empty(BG, gs, nc, dtype=torch.float32, device=dev)
    ret = torch.empty(BG, nprobe, dtype=torch.int32, device=dev)
    est = torch.empty(BG, es, dtype=torch.int32, device=dev)
    off = torch.empty(BG, nprobe + 1, dtype=torch.int32, device=dev)
    rows = torch.full((BG, max_pages * page), -1, dtype=torch.int32, device=dev)
    meta = torch.empty(BG, 4, dtype=torch.int32, device=dev)
    kernels.score_select(q.to(dev), cent.to(dev), None, size.to(dev), start.to(dev), logits, None, None, ret, est,
                         off, rows, meta, nprobe, es, page, max_pages, 1 / math.sqrt(128))
    torch.cuda.synchronize()
    assert meta.cpu()[:, 0].tolist() == [3, 3]
    assert meta.cpu()[:, 1].tolist() == [60, 60]
    assert meta.cpu()[:, 2].tolist() == [9, 9]


def test_score_select_rejects_bad_shapes(dev):
    from retrievalattention_amd import kernels
    q, cent = _mixture(1, 4, 64, 0)
    logits = torch.empty(1, 4, 64, dtype=torch.float32, device=dev)
    ret = torch.empty(1, 80, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError, match="invalid argument"):
        kernels.score_select(q.to(dev), cent.to(dev), None, None, None, logits, None, None, ret, None, None, None,
                             None, 80, 0, 8, 16, 1.0)   # nprobe > nc
    q, cent = _mixture(1, 4, 8192, 0)
    logits = torch.empty(1, 4, 8192, dtype=torch.float32, device=dev)
    ret = torch.empty(1, 4097, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError, match="invalid argument"):
        kernels.score_select(q.to(dev), cent.to(dev), None, None, None, logits, None, None, ret, None, None, None,
                             None, 4097, 0, 8, 16, 1.0)   # more probes than the selection lays out


def test_misaligned_rows_are_rejected(dev):
    """Rows are read 16 bytes at a time: a matrix that does not start on a 16-byte boundary is an
    invalid argument (nothing is launched)."""
    from retrievalattention_amd import kernels
    q, cent = _mixture(1, 4, 64, 0)
    flat = torch.empty(64 * 128 + 8, dtype=torch.bfloat16, device=dev)
    shifted = flat[1:1 + 64 * 128].view(1, 64, 128)          # 2 bytes off
    shifted.copy_(cent.to(dev))
    logits = torch.empty(1, 4, 64, dtype=torch.float32, device=dev)
    ret = torch.empty(1, 4, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError, match="invalid argument"):
        kernels.score_select(q.to(dev), shifted, None, None, None, logits, None, None, ret, None, None, None,
                             None, 4, 0, 8, 16, 1.0)
    k = torch.empty(1 * 40 * 128 + 8, dtype=torch.bfloat16, device=dev)[1:1 + 40 * 128].view(1, 40, 1, 128)
    with pytest.raises(RuntimeError, match="invalid argument"):
        kernels.weighted_flash_decoding(q.view(1, 1, 4, 128).to(dev), k, k)
