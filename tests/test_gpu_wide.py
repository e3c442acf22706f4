"""The wide permute-dot scan (every query of a chunk in one pass over the codes) against the
CPU oracle and against the tile-group kernels it replaces for large high-dimensional
batches.  Bar: slots and float scores bit-exact."""
import numpy as np
import pytest

from helpers import OracleIndex, bits_equal, ladder_for, to_native, unit_gaussian

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def T():
    from turbovec_amd import _lib
    _lib.lib()
    return _lib


def masks_for(T, n, seed):
    rng = np.random.default_rng(seed)
    out = [None, rng.random(n) < 0.5, rng.random(n) < 0.004, (np.arange(n) >= n // 3) & (np.arange(n) < n // 3 + 700)]
    return [None if m is None else T.pack_mask(m)[0] for m in out]


# dims 1280 to 2304 switch to the wide kernel at 97 queries (2048 and up: its four-wave form, a
# row's operands in 512 registers), dims up to 1024 and from 2560 at 129 (256 to 768: two to four blocks per wave); the query counts
# leave a ragged last tile, and 1029 = one full chunk of 1024 plus a 5-query chunk that the
# single-tile kernel serves
@pytest.mark.parametrize("dim,n,nq", [(1536, 6_007, 300), (1280, 4_001, 257), (1280, 3_001, 100), (1024, 5_003, 520), (1536, 3_001, 1029),
                                      (2048, 3_001, 200), (2560, 2_001, 140), (3072, 2_501, 260),
                                      (256, 20_011, 333), (384, 9_001, 130), (512, 12_345, 200), (768, 7_003, 290),
                                      (1024, 4_001, 129), (128, 30_011, 400), (640, 5_003, 140), (896, 4_001, 200),
                                      (1152, 3_001, 130), (1408, 3_003, 100), (1792, 2_001, 100), (2304, 2_003, 129),
                                      (2816, 1_501, 160),
                                      # row lengths that are not a whole number of chunk pairs: padded with zero
                                      # chunks to the next instance (1600: 25 -> 26 chunks, 2080: 33 -> 36,
                                      # 1000 and 200: partly filled last chunk)
                                      (1600, 3_001, 140), (2080, 2_001, 130), (1000, 4_001, 150), (200, 20_011, 333),
                                      (1736, 2_501, 129), (2952, 1_203, 131),
                                      # rows beyond one wave's registers (over 48 chunks): split over wave pairs
                                      (4096, 1_501, 131), (3584, 1_203, 260), (4104, 1_001, 129), (5000, 1_003, 150),
                                      (6144, 1_001, 140), (3200, 1_501, 1029),
                                      # more than 1024 queries at 1536 dimensions: one chunk of up to 1632 on the
                                      # ring of five slices, up to 2048 on the ring of nine; 2100 = 2048 + 52
                                      (1536, 2_001, 1500), (1536, 2_001, 1700), (1536, 1_501, 2100)])
def test_wide_scan_matches_oracle(T, oracle, dim, n, nq):
    oidx = OracleIndex(oracle, dim, 4, unit_gaussian(n, dim, seed=dim + n))
    q = unit_gaussian(nq, dim, seed=77)
    ix = to_native(T, oidx)
    for words in masks_for(T, n, 8):
        for k in (1, 10, 100):
            s, i = ix.search(q, k, mask_words=words)
            assert ix.queries_per_launch() == min(nq, 2048 if dim == 1536 else 1024)
            os_, oi = oidx.search(q, k, mask_words=words)
            assert np.array_equal(i, oi), k
            assert bits_equal(s, os_), k
    ix.close()


def test_rows_beyond_the_wide_kernel_fall_back_exactly(T, oracle):
    """More than 96 chunks (over 6144 dimensions at 4 bits): no all-queries-per-pass instance,
    the tile-group kernels serve the batch, results unchanged."""
    dim, n, nq = 6400, 1_001, 131
    oidx = OracleIndex(oracle, dim, 4, unit_gaussian(n, dim, seed=9))
    q = unit_gaussian(nq, dim, seed=10)
    ix = to_native(T, oidx)
    for words in masks_for(T, n, 8)[:2]:
        for k in (1, 10, 100):
            s, i = ix.search(q, k, mask_words=words)
            assert ix.queries_per_launch() < nq
            os_, oi = oidx.search(q, k, mask_words=words)
            assert np.array_equal(i, oi) and bits_equal(s, os_), k
    ix.close()


def test_wide_launch_covers_the_chunk(T, oracle):
    """The library reports how many queries its last full-scan launch served: the whole
    chunk on the wide path, at most a group of tiles with the wide path switched off."""
    oidx = OracleIndex(oracle, 1536, 4, unit_gaussian(2_000, 1536, seed=5))
    ix = to_native(T, oidx)
    q = unit_gaussian(512, 1536, seed=6)
    ix.search(q, 10)
    assert ix.queries_per_launch() == 512
    ix.set_path(4)
    ix.search(q, 10)
    assert ix.queries_per_launch() < 512
    ix.close()


# device-encoded index too large for the oracle: the wide kernel against the tile-group
# kernels and the exact full-list path on the same index (k up to the sort capacity's regime)
@pytest.mark.parametrize("dim,n,nq", [(1536, 300_000, 1024 + 300), (1024, 200_000, 700), (3072, 150_000, 1024),
                                      (256, 500_000, 1024), (768, 400_000, 600)])
def test_wide_scan_matches_other_paths(T, dim, n, nq):
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(dim)
    ix = T.NativeIndex(dim, 4)
    for c0 in range(0, n, 100_000):
        v = torch.randn(min(100_000, n - c0), dim, device=dev, generator=gen)
        torch.cuda.synchronize()
        ix.add_dev(v.data_ptr(), v.shape[0])
    q = torch.randn(nq, dim, device=dev, generator=gen).cpu().numpy()
    for words in masks_for(T, n, 9):
        for k in (10, 1000):
            s, i = ix.search(q, k, mask_words=words)
            ix.set_path(4)
            s2, i2 = ix.search(q, k, mask_words=words)
            ix.set_path(0)
            assert np.array_equal(i, i2) and bits_equal(s, s2), k
        ix.set_path(1)
        s3, i3 = ix.search(q[:40], 10, mask_words=words)
        ix.set_path(0)
        s, i = ix.search(q, 10, mask_words=words)
        assert np.array_equal(i[:40], i3) and bits_equal(s[:40], s3)
    ix.close()


def test_wide_scan_stops_early_when_every_query_overflows(T):
    """Rows laid out against the sampler for a whole batch: the one sampling level (8192 blocks,
    k=10: 1024 sampled slots, every 256th block: the stride is asked of the library) reads blocks
    that hold the opposite of what the queries look for, every other block near-duplicates of it.  Every query's candidate
    segments fill within a round, the workgroups of the all-queries-per-pass kernel stop claiming
    blocks, and the batch is scanned again from raised floors: the answer equals the exact path's
    and the tile-group kernels', and no query needs the exact path."""
    dev = torch.device("cuda:0")
    dim, n, nq = 256, 8192 * 32, 200
    gen = torch.Generator(device=dev)
    gen.manual_seed(5)
    c = torch.randn(dim, device=dev, generator=gen)
    c = c / c.norm()
    strides, _ = ladder_for(T, dim, 4, n, nq, 10)
    assert len(strides) == 2 and strides[1] == 1, strides
    stride = int(strides[0])
    ix = T.NativeIndex(dim, 4)
    for c0 in range(0, n, 65_536):
        m = min(65_536, n - c0)
        block = (torch.arange(c0, c0 + m, device=dev) // 32)
        sign = torch.where(block % stride == 0, -1.0, 1.0).unsqueeze(1)
        v = sign * c + 0.3 * torch.randn(m, dim, device=dev, generator=gen) / dim ** 0.5
        torch.cuda.synchronize()
        ix.add_dev(v.data_ptr(), m)
    q = (c + 0.3 * torch.randn(nq, dim, device=dev, generator=gen) / dim ** 0.5).cpu().numpy()
    s, i = ix.search(q, 10)
    assert ix.queries_per_launch() == nq
    assert ix.overflow_redos() >= nq and ix.exact_redos() == 0
    ix.set_path(4)                                     # tile-group kernels
    s2, i2 = ix.search(q, 10)
    ix.set_path(1)                                     # exact path
    s3, i3 = ix.search(q[:24], 10)
    ix.set_path(0)
    assert np.array_equal(i, i2) and bits_equal(s, s2)
    assert np.array_equal(i[:24], i3) and bits_equal(s[:24], s3)
    ix.close()


def test_wide_scan_with_wild_row_scales(T, oracle):
    """Row scales far from the encoder's (zeros, tiny, huge: the accumulator bound divides by the
    block's largest one) against the oracle; with negative ones mixed in (a foreign snapshot
    could hold them; such blocks skip the bound) against the tile-group and exact paths."""
    dim, n, nq = 1536, 5_003, 200
    oidx = OracleIndex(oracle, dim, 4, unit_gaussian(n, dim, seed=31))
    rng = np.random.default_rng(32)
    factors = rng.choice(np.array([0.0, 1e-12, 1e-3, 1.0, 3.7, 1e6], np.float32), size=n)
    oidx.scales = (oidx.scales * factors).astype(np.float32)
    q = unit_gaussian(nq, dim, seed=33)
    ix = to_native(T, oidx)
    for k in (1, 10, 100):
        s, i = ix.search(q, k)
        assert ix.queries_per_launch() == nq
        os_, oi = oidx.search(q, k)
        assert np.array_equal(i, oi) and bits_equal(s, os_), k
    ix.close()
    oidx.scales[rng.random(n) < 0.02] *= np.float32(-1.0)
    ix = to_native(T, oidx)
    for k in (10, 100):
        s, i = ix.search(q, k)
        ix.set_path(4)
        s2, i2 = ix.search(q, k)
        ix.set_path(1)
        s3, i3 = ix.search(q, k)
        ix.set_path(0)
        assert np.array_equal(i, i2) and bits_equal(s, s2), k
        assert np.array_equal(i, i3) and bits_equal(s, s3), k
    ix.close()


# batch_matches_single.rs / kernel_correctness.rs:268-312, for batches that take the wide kernel:
# every row of the batch equals the same query searched alone (another kernel), ids and score bits;
# query_scale_invariance.rs: ids survive a power-of-two scaling of the queries
def test_wide_batch_equals_single_and_scale_invariance(T, oracle):
    dim, n = 1536, 4_003
    oidx = OracleIndex(oracle, dim, 4, unit_gaussian(n, dim, seed=51))
    ix = to_native(T, oidx)
    q = unit_gaussian(130, dim, seed=52)
    s, i = ix.search(q, 10)
    assert ix.queries_per_launch() == 130
    for qi in range(0, 130, 7):
        s1, i1 = ix.search(q[qi:qi + 1], 10)
        assert np.array_equal(i1[0], i[qi]) and bits_equal(s1[0], s[qi])
    for e in (-60, -20, 10, 40):
        _, i2 = ix.search(q * np.float32(2.0 ** e), 10)
        assert np.array_equal(i2, i)
    ix.close()


# concurrent_search.rs: threads searching one index at once see identical results
def test_wide_concurrent_searches(T, oracle):
    import threading
    dim, n = 1280, 3_001
    oidx = OracleIndex(oracle, dim, 4, unit_gaussian(n, dim, seed=53))
    ix = to_native(T, oidx)
    q = unit_gaussian(150, dim, seed=54)
    want_s, want_i = ix.search(q, 10)
    bad = []

    def worker():
        for _ in range(6):
            s, i = ix.search(q, 10)
            if not (np.array_equal(i, want_i) and bits_equal(s, want_s)):
                bad.append(1)

    threads = [threading.Thread(target=worker) for _ in range(6)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not bad
    ix.close()


# seeded sweep over row lengths (with and without a wide-kernel instance), sizes the oracle
# cannot reach in seconds, batch sizes around the switch-over points, k around the selection
# paths' limits, norm spread, duplicate rows (ties) and masks: the three search paths -- all
# queries per pass, tile groups, exact lists / radix select -- must agree bit for bit
def test_paths_agree_on_random_shapes(T):
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(2024)
    dims = [128, 256, 384, 512, 640, 768, 896, 1024, 1152, 1280, 1408, 1536, 1792, 2048, 2304, 2560, 2816, 3072,
            320, 1600]
    for case in range(24):
        dim = int(rng.choice(dims))
        n = int(rng.integers(50, 120_000 if dim <= 1536 else 50_000))
        nq = int(rng.choice([97, 128, 129, 130, 200, 257, 333, 512, 777, 1024, 1025]))
        k = int(rng.choice([1, 10, 16, 64, 65, 100, 300]))
        gen = torch.Generator(device=dev)
        gen.manual_seed(case * 7919 + 1)
        ix = T.NativeIndex(dim, 4)
        v = torch.randn(n, dim, device=dev, generator=gen)
        if rng.random() < 0.3:
            v *= torch.exp(torch.randn(n, 1, device=dev, generator=gen))
        if rng.random() < 0.2:
            v[: n // 3] = v[n // 3: 2 * (n // 3)]
        torch.cuda.synchronize()
        ix.add_dev(v.data_ptr(), n)
        q = torch.randn(nq, dim, device=dev, generator=gen).cpu().numpy()
        kind = int(rng.integers(0, 4))
        m = None
        if kind == 1:
            m = rng.random(n) < rng.choice([0.5, 0.05, 0.002])
        elif kind == 2:
            lo = int(rng.integers(0, n))
            m = (np.arange(n) >= lo) & (np.arange(n) < lo + max(1, n // 20))
        elif kind == 3:
            m = np.zeros(n, bool)
            m[rng.integers(0, n, size=min(n, 7))] = True
        words = None if m is None else T.pack_mask(m)[0]
        res = []
        for path in (0, 4, 1):
            ix.set_path(path)
            res.append(ix.search(q, k, mask_words=words))
        for s, i in res[1:]:
            assert np.array_equal(res[0][1], i) and bits_equal(res[0][0], s), (case, dim, n, nq, k, kind)
        ix.close()
        del v


# the same for batches below the wide kernel's: the single-tile scan (one to 32 queries, every
# burst length of its sixteen-wave form, rows whose weights do not fit LDS), the resident-weights
# tile-group kernel (two to four tiles) and the streamed one (two to four tiles, from 2560
# dimensions) against the exact full-list path, bit for bit
def test_small_batches_agree_with_the_exact_path_on_random_shapes(T):
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(77)
    dims = [128, 192, 256, 320, 384, 512, 704, 768, 1024, 1280, 1472, 1536, 1792, 2048, 2560, 2624, 3072, 4096, 5120, 5376]
    for case in range(36):
        dim = int(rng.choice(dims))
        n = int(rng.integers(40, 90_000 if dim <= 1536 else 30_000))
        nq = int(rng.choice([1, 2, 7, 8, 9, 16, 31, 32, 33, 45, 64, 65, 70, 96, 97, 128]))
        k = int(rng.choice([1, 10, 16, 64, 100]))
        gen = torch.Generator(device=dev)
        gen.manual_seed(case * 104729 + 3)
        ix = T.NativeIndex(dim, 4)
        v = torch.randn(n, dim, device=dev, generator=gen)
        if rng.random() < 0.3:
            v *= torch.exp(torch.randn(n, 1, device=dev, generator=gen))
        if rng.random() < 0.2:
            v[: n // 3] = v[n // 3: 2 * (n // 3)]
        torch.cuda.synchronize()
        ix.add_dev(v.data_ptr(), n)
        q = torch.randn(nq, dim, device=dev, generator=gen).cpu().numpy()
        kind = int(rng.integers(0, 4))
        m = None
        if kind == 1:
            m = rng.random(n) < rng.choice([0.5, 0.05, 0.002])
        elif kind == 2:
            lo = int(rng.integers(0, n))
            m = (np.arange(n) >= lo) & (np.arange(n) < lo + max(1, n // 20))
        elif kind == 3:
            m = np.zeros(n, bool)
            m[rng.integers(0, n, size=min(n, 7))] = True
        words = None if m is None else T.pack_mask(m)[0]
        res = []
        for path in (0, 1):
            ix.set_path(path)
            res.append(ix.search(q, k, mask_words=words))
        assert np.array_equal(res[0][1], res[1][1]) and bits_equal(res[0][0], res[1][0]), (case, dim, n, nq, k, kind)
        ix.close()
        del v


# the tile-group kernel tests the same accumulator bound before it scores a tile in floats
@pytest.mark.parametrize("dim,nq", [(1536, 64), (1536, 96), (512, 128), (2048, 40)])
def test_tile_group_scan_with_wild_row_scales_and_query_scales(T, oracle, dim, nq):
    """Row scales far from the encoder's (zeros, tiny, huge, then negative ones mixed in) and queries
    scaled by powers of two far outside the unit range (floors and query scales beyond the range the
    bound is derived for switch it off) on batches the tile-group kernels serve: against the oracle,
    and against the exact path."""
    n = 5_003
    oidx = OracleIndex(oracle, dim, 4, unit_gaussian(n, dim, seed=61))
    rng = np.random.default_rng(62)
    factors = rng.choice(np.array([0.0, 1e-12, 1e-3, 1.0, 3.7, 1e6], np.float32), size=n)
    oidx.scales = (oidx.scales * factors).astype(np.float32)
    q = unit_gaussian(nq, dim, seed=63)
    ix = to_native(T, oidx)
    for k in (1, 10, 100):
        s, i = ix.search(q, k)
        assert 32 < ix.queries_per_launch() <= 128
        os_, oi = oidx.search(q, k)
        assert np.array_equal(i, oi) and bits_equal(s, os_), k
    for e in (-120, -60, 40, 100):
        qe = q * np.float32(2.0 ** e)
        s, i = ix.search(qe, 10)
        os_, oi = oidx.search(qe, 10)
        assert np.array_equal(i, oi) and bits_equal(s, os_), e
    ix.close()
    oidx.scales[rng.random(n) < 0.02] *= np.float32(-1.0)
    ix = to_native(T, oidx)
    for k in (10, 100):
        s, i = ix.search(q, k)
        ix.set_path(1)
        s3, i3 = ix.search(q, k)
        ix.set_path(0)
        assert np.array_equal(i, i3) and bits_equal(s, s3), k
    ix.close()
