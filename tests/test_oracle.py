"""Pins the CPU oracle itself: against the reference's own test oracles, library routines,
closed forms and brute force, chosen so that a dropped term, a wrong sign/index or a transposed
operand fails (CPU only)."""
import math

import numpy as np
import pytest
import torch

from oracle import attention, kmeans as okm, pipeline, scoring
from oracle.numerics import BF16_MIN, rb, bf16_ulp
from oracle.wavebuf import LruModel


def _r(shape, g, scale=1.0):
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


# ---------------------------------------------------------------- scoring
def test_softmax_matches_reference_test_oracle():
    """library/retroinfer/test/test_batch_gemm_softmax.py:9-18 (bmm -> /sqrt(d) -> softmax),
    atol 1e-3 as in the reference's assertion (:50)."""
    g = torch.Generator().manual_seed(0)
    q, c = _r((6, 4, 128), g), _r((6, 1032, 128), g)
    D, m, inv, soft = scoring.batch_gemm_softmax(q, c)
    ref = torch.softmax(torch.bmm(q.float(), c.float().transpose(1, 2)) / math.sqrt(128), dim=-1)
    assert torch.allclose(soft.float(), ref, atol=1e-3)
    # rows of the fp32 softmax sum to one; the transposed operand would not have this shape
    assert soft.shape == (6, 4, 1032)
    z = torch.exp((torch.bmm(q.double(), c.double().transpose(1, 2)) / math.sqrt(128)) - m.double()[..., None]).sum(-1)
    assert torch.allclose(1.0 / z.float(), inv, rtol=1e-5)


def test_softmax_uses_bf16_logits_for_the_final_value():
    """batch_gemm_softmax.h:237-243: the exponent argument is the bf16-rounded logit."""
    x = torch.tensor([[[1.0 + 2 ** -9, 0.0, -3.0]]], dtype=torch.float32)   # rounds down to 1.0 in bf16
    D, m, inv, soft = scoring.softmax_from_logits(x)
    assert float(D[0, 0, 0]) == 1.0
    z = torch.exp(x - x.max()).sum()
    expect = (torch.exp(torch.tensor(1.0) - x.max()) / z).to(torch.bfloat16)
    assert float(soft[0, 0, 0]) == float(expect)


def test_half_elements_round_to_half():
    """The 16-bit element type comes from the tensors (batch_gemm_softmax.cu:185-197 dispatches on it; the reference's
    harnesses default to fp16, simple_test.py:29).  Known answers that tell the two roundings apart: 1 + 2^-9 is a
    half but not a bfloat16; 1 + 2^-12 is neither and rounds to 1 in half; 70000 overflows half but not bfloat16."""
    x = torch.tensor([[[1.0 + 2 ** -9, 1.0 + 2 ** -12, 0.0, -3.0]]], dtype=torch.float32)
    D, m, inv, soft = scoring.softmax_from_logits(x, torch.float16)
    assert D.dtype == torch.float16 and soft.dtype == torch.float16
    assert float(D[0, 0, 0]) == 1.0 + 2 ** -9 and float(D[0, 0, 1]) == 1.0
    z = torch.exp(x - x.max()).sum()
    expect = (torch.exp(torch.tensor([1.0 + 2 ** -9, 1.0, 0.0, -3.0]) - x.max()) / z).to(torch.float16)
    assert torch.equal(soft[0, 0], expect)
    # score sum and mask value in half
    d = scoring.dist_from_softmax(torch.stack([soft[0, 0], soft[0, 0]])[None], torch.tensor([[False, False, True, False]]))
    assert d.dtype == torch.float16 and float(d[0, 2]) == torch.finfo(torch.float16).min == -65504.0
    assert float(d[0, 0]) == float((2 * soft[0, 0, 0].float()).to(torch.float16))
    # spacing of the two types
    from oracle.numerics import ulp16
    t = torch.tensor([1.0, 3.0, 2.0 ** -15, 1000.0])
    assert ulp16(t, torch.float16).tolist() == [2.0 ** -10, 2.0 ** -9, 2.0 ** -24, 0.5]
    assert ulp16(t, torch.bfloat16).tolist() == [2.0 ** -7, 2.0 ** -6, 2.0 ** -22, 4.0]
    # attention and k-means outputs carry the element type of their inputs
    g = torch.Generator().manual_seed(8)
    q, k, v = (torch.randn(*s, generator=g).to(torch.float16) for s in ((2, 4, 128), (2, 40, 128), (2, 40, 128)))
    out, _ = attention.weighted_flash_decoding(q, k, v)
    ref = torch.nn.functional.scaled_dot_product_attention(q.double(), k.double(), v.double())
    assert out.dtype == torch.float16 and torch.allclose(out.double(), ref, atol=1e-3)   # bf16 would need 8e-3
    cent = torch.randn(8, 128, generator=g).to(torch.float16)
    s = np.full((8, 128), 1.0 + 2 ** -9, dtype=np.float32)
    upd = okm.update(cent, s, np.array([1, 0, 2, 0, 0, 0, 0, 0], dtype=np.int32), False)
    assert upd.dtype == torch.float16 and float(upd[0, 0]) == 1.0 + 2 ** -9 and torch.equal(upd[1], cent[1])
    assert float(upd[2, 0]) == float(torch.tensor((1.0 + 2 ** -9) / 2).to(torch.float16))
    vs = okm.value_sum(torch.full((3, 128), 30000.0, dtype=torch.float16), np.array([0, 0, 0]), 2)
    assert vs.dtype == torch.float16 and bool(torch.isinf(vs[0]).all()) and bool((vs[1] == 0).all())   # 90000 > 65504


def test_score_interval_brackets_the_oracle_scores():
    """The interval the GPU score check uses is a float64 restatement with a 4e-6 relative tolerance: the oracle's
    fp32 pipeline must fall inside it, and the interval must be a single value for nearly every cluster (else it
    would pin nothing)."""
    from tests.parity import bf16_bits_i, score_interval, ulp_distance_bf16
    g = torch.Generator().manual_seed(5)
    x = torch.randn(3, 4, 6000, generator=g) * 2.0
    mask = torch.rand(3, 6000, generator=g) < 0.02
    d = scoring.dist_from_softmax(scoring.softmax_from_logits(x)[3], mask)
    lo, hi = score_interval(x, mask)
    b = bf16_bits_i(d)
    assert bool(((b >= bf16_bits_i(lo)) & (b <= bf16_bits_i(hi))).all())
    w = ulp_distance_bf16(lo, hi)
    assert int(w.max()) <= 2 and float((w > 0).float().mean()) < 0.01
    assert bool((lo[mask] == BF16_MIN).all()) and bool((hi[mask] == BF16_MIN).all())


def test_select_agrees_with_torch_topk_and_brute_force():
    """retroinfer_cache.py:572-574.  Values must equal torch.topk's; ids equal a brute-force
    sort by (-score, id)."""
    g = torch.Generator().manual_seed(1)
    soft = (torch.rand(5, 4, 300, generator=g) * 0.01).to(torch.bfloat16)
    mask = torch.rand(5, 300, generator=g) < 0.1
    dist = scoring.dist_from_softmax(soft, mask)
    assert bool((dist[mask] == BF16_MIN).all())
    assert torch.equal(dist[~mask], soft.float().sum(1).to(torch.bfloat16)[~mask])
    nprobe, es = 7, 40
    ret, est = scoring.select(dist, nprobe, es)
    top = torch.topk(dist.float(), nprobe + es, dim=-1, largest=True, sorted=True)
    for b in range(5):
        got = torch.cat([ret[b], est[b]])
        assert torch.equal(torch.sort(dist[b, got].float(), descending=True).values, top.values[b])
        brute = sorted(range(300), key=lambda c: (-float(dist[b, c]), c))
        assert ret[b].tolist() == brute[:nprobe]
        assert est[b].tolist() == sorted(brute[nprobe:nprobe + es])


def test_retrieval_layout_cutoff():
    """wave_buffer_cpu.cpp:207-216: stop before the first cluster that overflows the buffer."""
    size = torch.tensor([[20, 1, 8, 17, 3]], dtype=torch.int32)
    ret = torch.tensor([[0, 3, 1, 2, 4]])
    kept, offs = scoring.retrieval_layout(ret, size, 8, 7)   # pages 3, 3, 1 | next would be 8 > 7
    assert kept.tolist() == [3] and offs.tolist() == [[0, 20, 37, 38, 38, 38]]
    kept, offs = scoring.retrieval_layout(ret, size, 8, 100)
    assert kept.tolist() == [5] and offs[0, -1] == 49


# ---------------------------------------------------------------- attention closed forms
def test_attention_w1_is_softmax_attention():
    g = torch.Generator().manual_seed(2)
    q, k, v = _r((3, 4, 128), g), _r((3, 257, 128), g), _r((3, 257, 128), g)
    out, lse = attention.weighted_flash_decoding(q, k, v)
    ref = torch.nn.functional.scaled_dot_product_attention(q.double(), k.double(), v.double())
    assert torch.allclose(out.double(), ref, atol=8e-3)
    s = (q.double() @ k.double().transpose(1, 2)) / math.sqrt(128)
    assert torch.allclose(lse.double(), torch.logsumexp(s, -1), atol=1e-5)


def test_attention_merge_identity():
    """(ii) previous_out/previous_lse merge == attention over the concatenation."""
    g = torch.Generator().manual_seed(3)
    q, k, v = _r((2, 4, 128), g), _r((2, 300, 128), g), _r((2, 300, 128), g)
    oa, la = attention.weighted_flash_decoding(q, k[:, :120], v[:, :120])
    ob, _ = attention.weighted_flash_decoding(q, k[:, 120:], v[:, 120:], None, oa, la)
    oc, _ = attention.weighted_flash_decoding(q, k, v)
    assert torch.allclose(ob.float(), oc.float(), atol=1.6e-2)   # oa went through bf16


def test_estimation_exact_for_singletons_and_identical_keys():
    """(iii) one token per cluster and (iv) identical keys in a cluster: the weighted estimate
    equals exact attention.  A denominator without the weights, or weights on the numerator,
    breaks (iv)."""
    g = torch.Generator().manual_seed(4)
    q = _r((1, 4, 128), g)
    cent = _r((1, 50, 128), g)
    sizes = torch.randint(1, 7, (1, 50), generator=g)
    ks, vs, vsum = [], [], torch.zeros(1, 50, 128, dtype=torch.float64)
    for c in range(50):
        n = int(sizes[0, c])
        vals = _r((n, 128), g)
        ks.append(cent[0, c].expand(n, 128)); vs.append(vals); vsum[0, c] = vals.double().sum(0)
    exact, lse_exact = attention.weighted_flash_decoding(q, torch.cat(ks)[None], torch.cat(vs)[None])
    logits = scoring.logits_fp32(q, cent, 1 / math.sqrt(128))
    eo, el = attention.estimation(logits, torch.arange(50)[None], vsum, sizes.to(torch.bfloat16))
    assert torch.allclose(eo.float(), exact.float(), atol=1e-2)
    assert torch.allclose(el.float(), lse_exact, atol=1e-4)
    # same thing through the weighted call, as the reference issues it (retroinfer_cache.py:611-617)
    wo, wl = attention.weighted_flash_decoding(q, cent, vsum.to(torch.bfloat16), sizes.to(torch.bfloat16))
    assert torch.allclose(wo.float(), exact.float(), atol=2e-2)
    assert torch.allclose(wl, lse_exact, atol=1e-4)


def test_decode_step_full_probe_equals_dense_attention():
    """(v) nprobe = all clusters, no estimation zone: the pipeline is dense attention over
    steady zone + clustered tokens for any partition."""
    g = torch.Generator().manual_seed(5)
    BG, gs, n, nc = 2, 4, 400, 32
    keys, vals = _r((BG, n, 128), g), _r((BG, n, 128), g)
    q = _r((BG, gs, 128), g)
    steady_k, steady_v = _r((BG, 69, 128), g), _r((BG, 69, 128), g)
    a = torch.randint(0, nc, (BG, n), generator=g).numpy()
    size = torch.stack([torch.bincount(torch.from_numpy(a[b]), minlength=nc) for b in range(BG)]).to(torch.int32)
    sk, sv, st, cent = [], [], [], torch.zeros(BG, nc, 128)
    for b in range(BG):
        lists, cnt = okm.reverse_index(a[b], nc)
        k_, v_, s_ = pipeline.cluster_store(keys[b], vals[b], lists, size[b])
        sk.append(k_); sv.append(v_); st.append(s_)
    out, aux = pipeline.decode_step(q, steady_k, steady_v, 69, _r((BG, nc, 128), g), _r((BG, nc, 128), g),
                                    size == 0, size, size.to(torch.bfloat16), sk, sv, torch.stack(st), nc, 0, 8, 10 ** 6)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.double(), torch.cat([steady_k, keys], 1).double(), torch.cat([steady_v, vals], 1).double())
    assert torch.allclose(out.double(), ref, atol=8e-3)


# ---------------------------------------------------------------- k-means
def test_init_indices_follow_the_float32_formula():
    """kmeans.py:234-236: idx = int64(float32(i) * float32(N/nc) + float32(N/nc/2))."""
    for N, nc in ((131004, 8192), (8124, 512), (1000, 96)):
        idx = okm.init_indices(N, nc)
        step = np.float32(N / nc)
        expect = (np.arange(nc, dtype=np.float32) * step + np.float32(N / nc / 2)).astype(np.int64)
        assert np.array_equal(idx.numpy(), expect)
        assert idx[0] >= 0 and idx[-1] < N and bool((idx[1:] > idx[:-1]).all())


def test_assign_is_argmax_inner_product_with_first_index_ties():
    g = torch.Generator().manual_seed(6)
    data, cent = _r((200, 128), g), _r((40, 128), g)
    cent[17] = cent[5]                      # exact duplicate: the smaller id must win
    a, best, second = okm.assign(data, cent)
    s = data.double() @ cent.double().T
    for n in range(200):
        mx = float(s[n].max())
        assert float(s[n, a[n]]) == mx
        assert a[n] == min(c for c in range(40) if float(s[n, c]) == mx)
    assert 17 not in set(a.tolist())
    # inner product, not L2 distance: scaling a centroid up attracts tokens
    cent2 = cent.clone(); cent2[3] = (cent2[3].float() * 8).to(torch.bfloat16)
    a2, _, _ = okm.assign(data, cent2)
    assert (a2 == 3).sum() > (a == 3).sum()


def test_update_mean_normalise_and_empty_clusters():
    g = torch.Generator().manual_seed(7)
    data, cent = _r((300, 128), g), _r((16, 128), g)
    a = np.random.default_rng(0).integers(0, 12, 300)     # clusters 12..15 stay empty
    s, cnt = okm.cluster_sums(data, a, 16)
    assert int(cnt.sum()) == 300 and np.all(cnt[12:] == 0)
    ref_sum = np.stack([data[torch.from_numpy(a == c)].double().sum(0).numpy() for c in range(16)])
    assert np.allclose(s, ref_sum, rtol=1e-5, atol=1e-5)
    un = okm.update(cent, s, cnt, False)
    no = okm.update(cent, s, cnt, True)
    assert torch.equal(un[12:], cent[12:]) and torch.equal(no[12:], cent[12:])      # kmeans.py:75,80
    mean = ref_sum[:12] / cnt[:12, None]
    assert np.allclose(un[:12].float().numpy(), mean, rtol=1e-2, atol=1e-3)
    assert np.allclose(np.linalg.norm(no[:12].float().numpy(), axis=1), 1.0, atol=1e-2)
    assert np.allclose(no[:12].float().numpy(), mean / np.linalg.norm(mean, axis=1, keepdims=True), atol=1e-2)


def test_cluster_sums_blocked_order_by_brute_force():
    """The fixed summation order, restated as plain loops: blocks of 256 tokens in ascending
    index, one fp32 add per token from +0 inside a block, block sums added in block order."""
    g = torch.Generator().manual_seed(17)
    data = _r((1500, 128), g)
    a = np.random.default_rng(1).integers(0, 3, 1500)
    a[700:] = np.minimum(a[700:], 1)                        # cluster 1 grows past three blocks
    a[:40] = 5                                              # a short list; clusters 3, 4 stay empty
    s, cnt = okm.cluster_sums(data, a, 6)
    x = data.float().numpy()
    for c in range(6):
        ids = [n for n in range(1500) if a[n] == c]
        assert cnt[c] == len(ids)
        total = None
        for b in range(0, len(ids), okm.SUM_BLOCK):
            part = np.zeros(128, dtype=np.float32)
            for n in ids[b:b + okm.SUM_BLOCK]:
                part = (part + x[n]).astype(np.float32)
            total = part if total is None else (total + part).astype(np.float32)
        if total is None:
            total = np.zeros(128, dtype=np.float32)
        assert np.array_equal(s[c], total)
    assert max(cnt) > 2 * okm.SUM_BLOCK                     # the blocked path was exercised


def test_segment_k_means_invariants_and_remainder_tokens():
    """Each token in exactly one list; sizes add up; centroid * size = sum of keys (fp32 -> bf16);
    value_sum = sum of values; tokens past Nseg*S are only seen by the final pass."""
    g = torch.Generator().manual_seed(8)
    G, N, nc, S = 2, 1030, 64, 2
    key, val = _r((G, N, 128), g), _r((G, N, 128), g)
    cent, vsum, clusters, csize, assign = okm.segment_k_means(key, val, nc, 4, S)
    assert csize.sum().item() == G * N
    for h in range(G):
        seen = np.concatenate([clusters[h, c, :csize[h, c]].numpy() for c in range(nc)])
        assert np.array_equal(np.sort(seen), np.arange(N))
        for c in range(nc):
            ids = clusters[h, c, :csize[h, c]].long()
            assert bool((assign[h][ids.numpy()] == c).all())
            if len(ids):
                assert torch.allclose(cent[h, c].float() * len(ids), key[h, ids].float().sum(0), rtol=2e-2, atol=2e-2 * len(ids))
                assert torch.allclose(vsum[h, c].float(), val[h, ids].float().sum(0), rtol=1e-2, atol=3e-2)
    # remainder: with the final pass removed the last N - (N//S)*S tokens influence nothing
    key2 = key.clone(); key2[:, (N // S) * S:] = _r((G, N - (N // S) * S, 128), g)
    idx = okm.init_indices(N, nc)
    c1 = key[:, idx].clone(); c2 = key2[:, idx].clone()
    same_init = torch.equal(c1, c2)
    if same_init:
        nseg, ncs = N // S, nc // S
        for s_ in range(S):
            a1 = okm.train_step(key[0, s_ * nseg:(s_ + 1) * nseg], c1[0, s_ * ncs:(s_ + 1) * ncs], True)[0]
            a2 = okm.train_step(key2[0, s_ * nseg:(s_ + 1) * nseg], c2[0, s_ * ncs:(s_ + 1) * ncs], True)[0]
            assert torch.equal(a1, a2)


def test_prefill_index_hand_worked_case():
    """retroinfer_cache.py:416-432 on a case small enough to follow by hand (every number is exact in bf16).
    Eight tokens whose keys are 3 in every dimension except dimension 0, which holds 4 4 6 6 2 2 0 0:
    the mean is 3 everywhere, the centred keys are (1 1 3 3 -1 -1 -3 -3) e0.  Four centroids start at
    tokens 1 3 5 7 = (1, 3, -1, -3) e0.  First pass: every positive token scores highest on 3 e0 (cluster
    1), every negative one on -3 e0 (cluster 3); their normalised means are e0 and -e0, clusters 0 and 2
    are empty and keep e0 and -e0.  From then on clusters 0/1 tie and so do 2/3: the smaller id wins, so
    the positive tokens sit in cluster 0 and the negative ones in cluster 2, while 1 and 3 stay empty at
    e0 and -e0.  The last pass does not normalise: cluster 0 ends at 2 e0, cluster 2 at -2 e0.  With the
    mean added back dimension 0 of the four centroids reads 5 4 1 2 and every other dimension 3."""
    D = 128
    keys = torch.full((1, 8, D), 3.0)
    keys[0, :, 0] = torch.tensor([4.0, 4.0, 6.0, 6.0, 2.0, 2.0, 0.0, 0.0])
    vals = torch.arange(1.0, 9.0)[None, :, None].expand(1, 8, D).contiguous()
    idx = pipeline.prefill_index(keys.to(torch.bfloat16), vals.to(torch.bfloat16), 4, 1, num_iters=10)
    want = torch.full((1, 4, D), 3.0)
    want[0, :, 0] = torch.tensor([5.0, 4.0, 1.0, 2.0])
    assert torch.equal(idx["centroids"].float(), want)
    assert idx["size"].tolist() == [[4, 0, 4, 0]]
    assert idx["mask"].tolist() == [[False, True, False, True]]
    assert idx["size_bf16"].dtype == torch.bfloat16 and idx["size_bf16"].tolist() == [[4.0, 0.0, 4.0, 0.0]]
    assert idx["assign"].tolist() == [[0, 0, 0, 0, 2, 2, 2, 2]]
    vs = torch.zeros(1, 4, D)
    vs[0, 0], vs[0, 2] = 10.0, 26.0            # 1+2+3+4 and 5+6+7+8
    assert torch.equal(idx["value_sum"].float(), vs)
    assert idx["lists"][0, 0, :4].tolist() == [0, 1, 2, 3] and idx["lists"][0, 2, :4].tolist() == [4, 5, 6, 7]
    # the cluster-contiguous store of this index: cluster 0's tokens, then cluster 2's
    sk, sv, start = pipeline.cluster_store(keys[0], vals[0], idx["lists"][0].numpy(), idx["size"][0])
    assert start.tolist() == [0, 4, 4, 8] and torch.equal(sk, keys[0]) and torch.equal(sv, vals[0])


# ---------------------------------------------------------------- LRU model
def test_lru_model_invariants():
    rng = np.random.default_rng(0)
    sizes = rng.integers(0, 30, 64)
    m = LruModel(sizes, 8, 20, 24)
    for step in range(200):
        ids = rng.choice(64, 5, replace=False)
        hit, miss = m.access(ids)
        pages = 0
        expect_fit = []
        for c in ids:
            pages += (sizes[c] + 7) // 8
            if pages > 24:
                break
            expect_fit.append(c)
        assert sum(s for _, s, _ in hit) + sum(s for _, s, _ in miss) == sum(sizes[c] for c in expect_fit)
        assert all((c in m.resident) for c in m.hit_keys) and all((c not in m.resident) for c in m.miss_keys)
        upd = m.update()
        blocks = [b for v in m.resident.values() for b in v]
        assert len(blocks) == len(set(blocks)) <= 20
        assert set(m.lru) == set(m.resident)
