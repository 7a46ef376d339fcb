"""K-means kernels against the oracle (GPU).

Assignment scores come out of the matrix cores, whose accumulation order differs from any CPU
sum, so a token may legitimately land on the runner-up centroid when the two best scores are
closer than fp32 rounding noise; the test accepts exactly that and nothing else.  Everything
downstream of the assignment (lists, sums, means, normalisation, value sums) is bit-exact."""
import numpy as np
import pytest
import torch

from oracle import kmeans as okm

pytestmark = pytest.mark.gpu


def _mixture(G, N, K, seed, sigma=0.3, dt=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    centers = torch.randn(G, K, 128, generator=g)
    a = torch.randint(K, (G, N), generator=g)
    keys = torch.gather(centers, 1, a[..., None].expand(G, N, 128)) + sigma * torch.randn(G, N, 128, generator=g)
    vals = torch.randn(G, N, 128, generator=g)
    return keys.to(dt), vals.to(dt)


def _check_assign(data, cent, got):
    """got must be the oracle's argmax, or a centroid whose fp64 score is within fp32 noise of it."""
    a, best, _ = okm.assign(data, cent)
    got = got.astype(np.int64)
    diff = np.nonzero(a != got)[0]
    if diff.size:
        s = (data[diff].double().numpy() * cent[got[diff]].double().numpy()).sum(1)
        scale = np.abs(data[diff].double().numpy()).sum(1) * np.abs(cent.double().numpy()).max()
        assert np.all(best[diff] - s <= 1e-6 * np.maximum(scale, 1.0)), "assignment differs beyond a near-tie"
    return diff.size


@pytest.mark.parametrize("P,N,nc,seed", [(3, 1000, 64, 0), (2, 8192, 512, 1), (1, 4100, 1024, 2), (4, 37, 32, 3)])
def test_assign_update_valuesum(dev, P, N, nc, seed, dt=torch.bfloat16):
    from retrievalattention_amd import kernels
    keys, vals = _mixture(P, N, nc, seed, dt=dt)
    idx = okm.init_indices(N, nc)
    cent = keys[:, idx].contiguous()
    kd, vd, cd = keys.to(dev), vals.to(dev), cent.to(dev).clone()
    assign = torch.empty(P, N, dtype=torch.int32, device=dev)
    counts = torch.empty(P, nc, dtype=torch.int32, device=dev)
    offsets = torch.empty(P, nc + 1, dtype=torch.int32, device=dev)
    members = torch.empty(P, N, dtype=torch.int32, device=dev)
    vsum = torch.empty(P, nc, 128, dtype=dt, device=dev)
    kernels.kmeans_assign(kd, cd, assign, P, N, nc, 1, N)
    kernels.kmeans_build_lists(assign, counts, offsets, members, P, N, nc)
    cn = cd.clone()
    kernels.kmeans_update(kd, counts, offsets, members, cn, P, N, nc, 1, N, True)
    cu = cd.clone()
    kernels.kmeans_update(kd, counts, offsets, members, cu, P, N, nc, 1, N, False)
    kernels.kmeans_value_sum(vd, counts, offsets, members, vsum, P, N, nc)
    torch.cuda.synchronize()
    A = assign.cpu().numpy()
    for p in range(P):
        _check_assign(keys[p], cent[p], A[p])
        # lists: counts, offsets and ascending members of the kernel's own assignment
        lists, cnt = okm.reverse_index(A[p].astype(np.int64), nc)
        assert np.array_equal(counts[p].cpu().numpy(), cnt)
        off = offsets[p].cpu().numpy()
        assert off[0] == 0 and np.array_equal(np.diff(off), cnt)
        mem = members[p].cpu().numpy()
        for c in range(nc):
            assert np.array_equal(mem[off[c]:off[c + 1]], lists[c, :cnt[c]])
        # sums / means / normalisation given that assignment: bit-exact
        s, cnt2 = okm.cluster_sums(keys[p], A[p].astype(np.int64), nc)
        assert torch.equal(cn[p].cpu(), okm.update(cent[p], s, cnt2, True))
        assert torch.equal(cu[p].cpu(), okm.update(cent[p], s, cnt2, False))
        assert torch.equal(vsum[p].cpu(), okm.value_sum(vals[p], A[p].astype(np.int64), nc))


@pytest.mark.parametrize("P,N,nc,seed", [(3, 1000, 64, 10), (2, 8192, 512, 11), (1, 4100, 1024, 12), (4, 37, 32, 13)])
def test_assign_update_valuesum_float16(dev, P, N, nc, seed):
    """IEEE half keys, values and centroids (the reference's harnesses default to fp16, simple_test.py:29):
    the same fixed-order fp32 sums, rounded to fp16 on store."""
    test_assign_update_valuesum(dev, P, N, nc, seed, dt=torch.float16)


def test_big_and_empty_clusters(dev):
    """All tokens identical: one cluster takes everything (list longer than a wave and than
    the LDS sort), the others stay empty and keep their centroid."""
    from retrievalattention_amd import kernels
    P, N, nc = 1, 20000, 64
    g = torch.Generator().manual_seed(5)
    row = torch.randn(128, generator=g).to(torch.bfloat16)
    keys = row.expand(P, N, 128).contiguous()
    cent = torch.randn(P, nc, 128, generator=g).to(torch.bfloat16)
    kd, cd = keys.to(dev), cent.to(dev).clone()
    assign = torch.empty(P, N, dtype=torch.int32, device=dev)
    counts = torch.empty(P, nc, dtype=torch.int32, device=dev)
    offsets = torch.empty(P, nc + 1, dtype=torch.int32, device=dev)
    members = torch.empty(P, N, dtype=torch.int32, device=dev)
    kernels.kmeans_assign(kd, cd, assign, P, N, nc, 1, N)
    kernels.kmeans_build_lists(assign, counts, offsets, members, P, N, nc)
    kernels.kmeans_update(kd, counts, offsets, members, cd, P, N, nc, 1, N, True)
    torch.cuda.synchronize()
    a, _, _ = okm.assign(keys[0, :1], cent[0])
    assert int(counts.cpu()[0, a[0]]) == N and int(counts.cpu().sum()) == N
    assert torch.equal(members.cpu()[0], torch.arange(N, dtype=torch.int32))
    keep = torch.ones(nc, dtype=torch.bool); keep[a[0]] = False
    assert torch.equal(cd.cpu()[0, keep], cent[0, keep])
    s, cnt = okm.cluster_sums(keys[0], np.full(N, a[0]), nc)
    assert torch.equal(cd.cpu()[0], okm.update(cent[0], s, cnt, True))


def test_medium_clusters_sorted(dev):
    """Clusters of a few hundred to a few thousand tokens exercise the workgroup sort."""
    from retrievalattention_amd import kernels
    P, N, nc = 2, 30000, 32
    g = torch.Generator().manual_seed(6)
    assign = torch.randint(0, 8, (P, N), generator=g, dtype=torch.int32)
    assign[0, ::3] = 31
    ad = assign.to(dev)
    counts = torch.empty(P, nc, dtype=torch.int32, device=dev)
    offsets = torch.empty(P, nc + 1, dtype=torch.int32, device=dev)
    members = torch.empty(P, N, dtype=torch.int32, device=dev)
    kernels.kmeans_build_lists(ad, counts, offsets, members, P, N, nc)
    torch.cuda.synchronize()
    for p in range(P):
        order = np.argsort(assign[p].numpy(), kind="stable")
        assert np.array_equal(members[p].cpu().numpy(), order.astype(np.int32))


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_long_lists_blocked_sums(dev, dt):
    """Lists of 1 to several thousand random rows: update and value sums equal the oracle's
    blocked fixed-order sums bit for bit (lists over 256 rows take the block-item path, several
    of them per problem, next to short lists and empty clusters)."""
    from retrievalattention_amd import kernels
    P, N, nc = 3, 20011, 96
    g = torch.Generator().manual_seed(16)
    keys = torch.randn(P, N, 128, generator=g).to(dt)
    vals = torch.randn(P, N, 128, generator=g).to(dt)
    assign = torch.randint(0, 5, (P, N), generator=g, dtype=torch.int32)       # five lists of ~4000
    small = torch.randint(8, 90, (P, N), generator=g, dtype=torch.int32)       # the rest: ~100 each, 90..95 empty
    pick = torch.rand(P, N, generator=g) < 0.4
    assign[pick] = small[pick]
    assign[1, :700] = 7                                                        # 700+: three blocks, last one ragged
    assign[2, 5] = 95                                                          # a single-row list
    cent = torch.randn(P, nc, 128, generator=g).to(dt)
    ad, kd, vd = assign.to(dev), keys.to(dev), vals.to(dev)
    counts = torch.empty(P, nc, dtype=torch.int32, device=dev)
    offsets = torch.empty(P, nc + 1, dtype=torch.int32, device=dev)
    members = torch.empty(P, N, dtype=torch.int32, device=dev)
    kernels.kmeans_build_lists(ad, counts, offsets, members, P, N, nc)
    for normalize in (True, False):
        cd = cent.to(dev).clone()
        kernels.kmeans_update(kd, counts, offsets, members, cd, P, N, nc, 1, N, normalize)
        vs = torch.full((P, nc, 128), 7.0, dtype=dt, device=dev)
        kernels.kmeans_value_sum(vd, counts, offsets, members, vs, P, N, nc)
        torch.cuda.synchronize()
        for p in range(P):
            a = assign[p].numpy().astype(np.int64)
            s, cnt = okm.cluster_sums(keys[p], a, nc)
            assert np.array_equal(counts[p].cpu().numpy(), cnt)
            assert torch.equal(cd[p].cpu(), okm.update(cent[p], s, cnt, normalize))
            assert torch.equal(vs[p].cpu(), okm.value_sum(vals[p], a, nc))


def test_long_lists_back_to_back(dev):
    """Long lists placed so that their blocks sit as close together as the layout allows (lengths
    just above one, two and three blocks, at offsets just below and at block boundaries, with empty
    and one-row clusters between and after them): every block is summed exactly once, in order."""
    from retrievalattention_amd import kernels
    sizes = [[255, 257, 0, 257, 1, 511, 0, 0, 512, 513, 255, 769, 3, 0, 300, 0],
             [0, 0, 1025, 1, 257, 257, 257, 0, 2, 256, 256, 258, 254, 768, 0, 0],
             [4000, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 257]]
    P, nc = len(sizes), 32
    N = max(sum(r) for r in sizes)
    g = torch.Generator().manual_seed(21)
    assign = torch.empty(P, N, dtype=torch.int32)
    for p, row in enumerate(sizes):
        row = row + [0] * (nc - len(row))
        row[nc - 2] += N - sum(row)                      # the remainder goes to one late cluster
        ids = torch.repeat_interleave(torch.arange(nc, dtype=torch.int32), torch.tensor(row))
        assign[p] = ids[torch.randperm(N, generator=g)]
    keys = torch.randn(P, N, 128, generator=g).to(torch.bfloat16)
    cent = torch.randn(P, nc, 128, generator=g).to(torch.bfloat16)
    ad, kd, cd = assign.to(dev), keys.to(dev), cent.to(dev).clone()
    counts = torch.empty(P, nc, dtype=torch.int32, device=dev)
    offsets = torch.empty(P, nc + 1, dtype=torch.int32, device=dev)
    members = torch.empty(P, N, dtype=torch.int32, device=dev)
    kernels.kmeans_build_lists(ad, counts, offsets, members, P, N, nc)
    kernels.kmeans_update(kd, counts, offsets, members, cd, P, N, nc, 1, N, True)
    vs = torch.full((P, nc, 128), 7.0, dtype=torch.bfloat16, device=dev)
    kernels.kmeans_value_sum(kd, counts, offsets, members, vs, P, N, nc)
    torch.cuda.synchronize()
    for p in range(P):
        a = assign[p].numpy().astype(np.int64)
        s, cnt = okm.cluster_sums(keys[p], a, nc)
        assert np.array_equal(counts[p].cpu().numpy(), cnt)
        assert torch.equal(cd[p].cpu(), okm.update(cent[p], s, cnt, True))
        assert torch.equal(vs[p].cpu(), okm.value_sum(keys[p], a, nc))


@pytest.mark.parametrize("P,N,nc,seed", [(3, 1000, 64, 0), (2, 16384, 512, 1), (2, 16385, 512, 2), (5, 37, 32, 3),
                                         (2, 8192, 512, 4), (1, 4100, 1024, 5), (2, 1023, 96, 6), (1, 1, 32, 7)])
def test_build_lists_is_a_stable_sort(dev, P, N, nc, seed):
    """Inverted lists over the sizes on either side of the single-workgroup path (problems of at most
    16384 tokens with at most 512 clusters) and of the one- and two-pass paths: members are the stable
    argsort of the assignment, offsets and counts its CSR bounds; some clusters are empty."""
    from retrievalattention_amd import kernels
    g = torch.Generator().manual_seed(seed)
    assign = torch.randint(0, max(nc - 3, 1), (P, N), generator=g, dtype=torch.int32)
    assign[0, N // 2:] = nc - 1                     # one long run, and the highest id in use
    ad = assign.to(dev)
    counts = torch.full((P, nc), -1, dtype=torch.int32, device=dev)
    offsets = torch.full((P, nc + 1), -1, dtype=torch.int32, device=dev)
    members = torch.full((P, N), -1, dtype=torch.int32, device=dev)
    kernels.kmeans_build_lists(ad, counts, offsets, members, P, N, nc)
    torch.cuda.synchronize()
    for p in range(P):
        a = assign[p].numpy()
        cnt = np.bincount(a, minlength=nc)
        assert np.array_equal(members[p].cpu().numpy(), np.argsort(a, kind="stable"))
        assert np.array_equal(counts[p].cpu().numpy(), cnt)
        assert np.array_equal(offsets[p].cpu().numpy(), np.concatenate([[0], np.cumsum(cnt)]))


@pytest.mark.parametrize("G,N,nc,S,seed", [(2, 4096, 256, 4, 0), (1, 8192, 512, 1, 1), (2, 3001, 192, 3, 2)])
def test_segment_k_means_teacher_forced(dev, G, N, nc, S, seed, dt=torch.bfloat16):
    """Whole driver against the oracle, iteration by iteration: every step is checked on the
    state the kernels actually produced (the trajectory itself is chaotic under near-ties)."""
    from retrievalattention_amd import kernels
    from retrievalattention_amd.cache_hub.kmeans import segment_k_means, segment_k_means_csr, csr_to_dense
    keys, vals = _mixture(G, N, nc, seed, dt=dt)
    kd, vd = keys.to(dev), vals.to(dev)
    cent, vsum, clusters, csize = segment_k_means(kd, vd, nc, 10, S)
    torch.cuda.synchronize()
    # replay with the kernels step by step, comparing each step with the oracle
    idx = okm.init_indices(N, nc)
    c_dev = kd[:, idx.to(dev)].contiguous()
    nseg, ncs, P = N // S, nc // S, G * S
    a = torch.empty(P, nseg, dtype=torch.int32, device=dev)
    cnt = torch.empty(P, ncs, dtype=torch.int32, device=dev)
    off = torch.empty(P, ncs + 1, dtype=torch.int32, device=dev)
    mem = torch.empty(P, nseg, dtype=torch.int32, device=dev)
    for it in range(9):
        before = c_dev.cpu().view(P, ncs, 128).clone()
        kernels.kmeans_assign(kd, c_dev, a, P, nseg, ncs, S, N)
        kernels.kmeans_build_lists(a, cnt, off, mem, P, nseg, ncs)
        kernels.kmeans_update(kd, cnt, off, mem, c_dev, P, nseg, ncs, S, N, True)
        torch.cuda.synchronize()
        A = a.cpu().numpy()
        after = c_dev.cpu().view(P, ncs, 128)
        for p in range(P):
            gi, si = p // S, p % S
            d = keys[gi, si * nseg:(si + 1) * nseg]
            _check_assign(d, before[p], A[p])
            s, c2 = okm.cluster_sums(d, A[p].astype(np.int64), ncs)
            assert torch.equal(after[p], okm.update(before[p], s, c2, True)), f"iteration {it} problem {p}"
    # final pass and outputs of the driver equal the replayed state
    r = segment_k_means_csr(kd, vd, nc, 10, S)
    torch.cuda.synchronize()
    assert torch.equal(r.centroids.cpu(), cent.cpu())
    before = c_dev.cpu()
    A = r.assign.cpu().numpy()
    for gi in range(G):
        _check_assign(keys[gi], before[gi], A[gi])
        s, c2 = okm.cluster_sums(keys[gi], A[gi].astype(np.int64), nc)
        assert torch.equal(cent.cpu()[gi], okm.update(before[gi], s, c2, False))
        assert torch.equal(vsum.cpu()[gi], okm.value_sum(vals[gi], A[gi].astype(np.int64), nc))
        lists, sz = okm.reverse_index(A[gi].astype(np.int64), nc)
        assert np.array_equal(csize.cpu().numpy()[gi], sz)
        assert np.array_equal(clusters.cpu().numpy()[gi][:, :lists.shape[1]], lists)
    # invariants: every token in exactly one list, sizes add up
    assert int(csize.sum()) == G * N


@pytest.mark.parametrize("G,N,nc,S,seed", [(2, 4096, 256, 4, 10), (2, 3001, 192, 3, 12)])
def test_segment_k_means_teacher_forced_float16(dev, G, N, nc, S, seed):
    test_segment_k_means_teacher_forced(dev, G, N, nc, S, seed, dt=torch.float16)
