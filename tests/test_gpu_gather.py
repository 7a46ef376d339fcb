"""Copy kernels against the loop oracles of library/retroinfer/test/test_gather_copy.py
(same shapes and edge cases: a group with no misses, one with no hits, a copy that ends on
the last vector of the source, zero-length blocks).  Bit-exact."""
import numpy as np
import pytest
import torch

from oracle import wavebuf as owb

pytestmark = pytest.mark.gpu
DT = torch.bfloat16


def _two_index_sets(rows, cols, max_range1, max_range2, unit, rng):
    """Random miss/hit lists in the layout of test_gather_copy.py:11-66."""
    def empty():
        return (rng.integers(-1, 100, (rows, cols)).astype(np.int32), rng.integers(1, unit + 1, (rows, cols)).astype(np.int32),
                rng.integers(0, 100, (rows, cols)).astype(np.int32), rng.integers(0, 10, (rows,)).astype(np.int32))
    i1, s1, d1, n1 = empty()
    i2, s2, d2, n2 = empty()
    for r in range(rows):
        num = int(rng.integers(int(0.8 * cols), cols))
        a = 0 if r == 1 else (num if r == 5 else int(rng.integers(0, num)))
        b = num - a
        i1[r, :a] = rng.choice(max_range1, a, replace=False)
        cs = 0
        for j in range(a):
            s1[r, j] = rng.integers(0, unit + 1); d1[r, j] = cs; cs += s1[r, j]
        if a > 0:
            x = int(rng.integers(0, a))
            i1[r, x] = max_range1 + unit - s1[r, x]   # copy that ends exactly at the end of the source
        n1[r] = a
        i2[r, :b] = rng.choice(max_range2, b, replace=False)
        cs = 0
        for j in range(b):
            s2[r, j] = rng.integers(0, unit + 1); d2[r, j] = cs; cs += s2[r, j]
        n2[r] = b
    pin = lambda a: torch.from_numpy(a).pin_memory()
    return [pin(t) for t in (i1, s1, d1, n1, i2, s2, d2, n2)]


@pytest.mark.parametrize("seed", [0, 1])
def test_concat_gather_copy(dev, seed):
    from retrievalattention_amd import kernels
    rng = np.random.default_rng(seed)
    torch.manual_seed(seed)
    groups, n1, n2, units3, buf_units, idx_len, unit, dim, copy1 = 8, 1769, 12397, 1000, 400, 400, 8, 128, 1602
    buf = buf_units * unit + n1
    k1 = torch.randn(groups, n1, dim).to(DT).to(dev); v1 = torch.randn(groups, n1, dim).to(DT).to(dev)
    k2 = torch.randn(groups, n2, dim).to(DT).pin_memory(); v2 = torch.randn(groups, n2, dim).to(DT).pin_memory()
    k3 = torch.randn(groups, units3, unit, dim).to(DT).to(dev); v3 = torch.randn(groups, units3, unit, dim).to(DT).to(dev)
    kd = torch.randn(groups, buf, dim).to(DT).to(dev); vd = torch.randn(groups, buf, dim).to(DT).to(dev)
    kd2, vd2 = kd.cpu().clone(), vd.cpu().clone()
    valid = torch.empty(groups, dtype=torch.int32).pin_memory()
    o2, s2, d2, c2, o3, s3, d3, c3 = _two_index_sets(groups, idx_len, n2 - unit, units3, unit, rng)
    kernels.gather_copy_and_concat(k1, k2, k3, kd, v1, v2, v3, vd, o2, s2, d2, c2, o3, s3, d3, c3, valid,
                                   groups, n1, n2, units3, buf, idx_len, copy1)
    torch.cuda.synchronize()
    ref_valid = owb.concat_gather(kd2, vd2, k1.cpu(), v1.cpu(), k2, v2, k3.cpu(), v3.cpu(), o2, s2, c2, o3, s3, c3, copy1)
    assert valid.tolist() == ref_valid
    assert torch.equal(kd.cpu(), kd2) and torch.equal(vd.cpu(), vd2)


@pytest.mark.parametrize("seed", [0, 1])
def test_gather_copy_scatter(dev, seed):
    from retrievalattention_amd import kernels
    rng = np.random.default_rng(seed)
    torch.manual_seed(seed)
    groups, src_units, dst_units, idx_len, unit, dim, start = 8, 400, 1000, 400, 8, 128, 97
    ks = torch.randn(groups, src_units * unit, dim).to(DT).to(dev); vs = torch.randn(groups, src_units * unit, dim).to(DT).to(dev)
    kc = torch.randn(groups, dst_units, unit, dim).to(DT).to(dev); vc = torch.randn(groups, dst_units, unit, dim).to(DT).to(dev)
    kc2, vc2 = kc.cpu().clone(), vc.cpu().clone()
    max1 = src_units * unit - start
    so = rng.integers(-1, 100, (groups, idx_len)).astype(np.int32)
    sz = rng.integers(1, unit + 1, (groups, idx_len)).astype(np.int32)
    do = rng.integers(0, 100, (groups, idx_len)).astype(np.int32)
    num = rng.integers(0, 10, (groups,)).astype(np.int32)
    for r in range(groups):
        if r == 1:
            num[r] = 0
            continue
        n = int(rng.integers(int(0.2 * idx_len), int(0.8 * idx_len)))
        so[r, :n] = rng.choice(max1, n, replace=False)
        do[r, :n] = rng.choice(dst_units, n, replace=False)
        for j in range(n):
            s = int(rng.integers(0, unit + 1))
            sz[r, j] = min(s, max1 - so[r, j])
        num[r] = n
    pin = lambda a: torch.from_numpy(a).pin_memory()
    so, sz, do, num = pin(so), pin(sz), pin(do), pin(num)
    kernels.gather_copy_and_scatter(ks, kc, vs, vc, so, sz, do, num, groups, src_units * unit, dst_units, idx_len, start)
    torch.cuda.synchronize()
    owb.gather_scatter(kc2, vc2, ks.cpu(), vs.cpu(), so, sz, do, num, start)
    assert torch.equal(kc.cpu(), kc2) and torch.equal(vc.cpu(), vc2)


@pytest.mark.parametrize("DT", [torch.bfloat16, torch.float16])
def test_gather_copy_vectors(dev, DT):
    """Half and BFloat16, the two element types gather_copy.cu:63-67 accepts."""
    from retrievalattention_amd import kernels
    torch.manual_seed(3)
    groups, n, dim, nprobe, idx_size = 8, 8192, 128, 150, 2048
    num = idx_size - nprobe
    ks = torch.randn(groups, n, dim).to(DT).to(dev); vs = torch.randn(groups, n, dim).to(DT).to(dev)
    ms = torch.randn(groups, n).to(DT).to(dev)
    kd = torch.randn(groups, num, dim).to(DT).to(dev); vd = torch.randn(groups, num, dim).to(DT).to(dev)
    md = torch.empty(groups, num, dtype=DT, device=dev)
    idx = torch.stack([torch.randperm(n)[:idx_size] for _ in range(groups)]).to(torch.int64)
    kernels.gather_copy_vectors(ks, kd, vs, vd, ms, md, idx.to(dev), groups, n, num, idx_size, nprobe, num)
    torch.cuda.synchronize()
    rk, rv, rm = owb.gather_copy_vectors(ks.cpu(), vs.cpu(), ms.cpu(), idx, nprobe, num)
    assert torch.equal(kd.cpu(), rk) and torch.equal(vd.cpu(), rv) and torch.equal(md.cpu(), rm)
