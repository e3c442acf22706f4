"""Rows laid out against the sampling ladder, calls merged across threads, calls of several
chunks, and queries the caller should have refused: the answer must stay the oracle's (or the
exact path's), bit for bit, whatever route the search takes to it."""
import threading

import numpy as np
import pytest

from helpers import OracleIndex, bits_equal, ladder_for, to_native, unit_gaussian

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def T():
    from turbovec_amd import _lib
    _lib.lib()
    return _lib


def rows_against(strides_poisoned, n, dim, u, seed):
    """Rows near +u, except in the blocks the given strides sample (multiples of any of them): those
    point away from u, so a level that reads only them sees nothing worth keeping."""
    rng = np.random.default_rng(seed)
    block = np.arange(n) // 32
    bad = np.zeros(n, bool)
    for s in strides_poisoned:
        bad |= block % int(s) == 0
    v = np.where(bad, -1.0, 1.0)[:, None].astype(np.float32) * (0.3 * u) + \
        rng.standard_normal((n, dim), dtype=np.float32) / np.float32(dim ** 0.5)
    return v / np.linalg.norm(v, axis=1, keepdims=True).astype(np.float32)


def queries_near(u, nq, dim, seed):
    rng = np.random.default_rng(seed)
    q = u + 0.5 * rng.standard_normal((nq, dim), dtype=np.float32) / np.float32(dim ** 0.5)
    return q / np.linalg.norm(q, axis=1, keepdims=True).astype(np.float32)


# 64 queries: the tile-group kernel; 140: every query in one pass; 2-bit: the LUT scan.  (Up to 32
# queries of a 4-bit index take the single-tile kernel, whose ladder has one sampling level only.)
@pytest.mark.parametrize("bits,nq", [(4, 64), (4, 140), (2, 4)])
def test_first_level_poisoned_repeats_the_second_level_only(T, oracle, bits, nq):
    """300,000 rows, k=10: the ladder is 1/293 of the blocks, then 1/17, then all.  The blocks of the
    first level hold rows pointing away from the queries, all others rows pointing towards them:
    the first floor lets every row of the second level through, its candidates overflow, and the
    level runs again from the floor taken from what fitted.  The full scan then starts from a good
    floor: no query is scanned twice, and the answer is the oracle's."""
    dim, n, k = 128, 300_000, 10
    rng = np.random.default_rng(1)
    u = rng.standard_normal(dim).astype(np.float32)
    u /= np.linalg.norm(u)
    strides, _ = ladder_for(T, dim, bits, n, nq, k)
    assert len(strides) == 3 and strides[-1] == 1, strides
    oidx = OracleIndex(oracle, dim, bits, rows_against(strides[:1], n, dim, u, seed=2))
    q = queries_near(u, nq, dim, seed=3)
    ix = to_native(T, oidx)
    ix.level_repeats(track=1)
    s, i = ix.search(q, k)
    assert ix.level_repeats() >= 1, "the layout did not overflow the second level: the test tests nothing"
    assert ix.overflow_redos() == 0 and ix.exact_redos() == 0
    os_, oi = oracle.search_fast(oidx.rot, oidx.seq, oidx.scales, q, k, bits, dim, n)
    assert np.array_equal(i, oi) and bits_equal(s, os_)
    ix.close()


# 8 queries: the single-tile kernel, whose one sampling level keeps the best row of every block it reads;
# 2-bit, 20 queries: the sixteen-query LUT scan (tiles of 16 and 4), first and repeated pass
@pytest.mark.parametrize("bits,nq", [(4, 8), (4, 140), (2, 20)])
def test_every_level_poisoned_goes_through_the_repeated_pass(T, oracle, bits, nq):
    """Every block any level of the first pass reads is poor: the full scan starts from a hopeless
    floor, every query overflows, the batch is scanned again from raised floors with the ladder
    shifted half a stride, and still equals the oracle."""
    dim, n, k = 128, 300_000, 10
    rng = np.random.default_rng(4)
    u = rng.standard_normal(dim).astype(np.float32)
    u /= np.linalg.norm(u)
    strides, offsets = ladder_for(T, dim, bits, n, nq, k)
    assert len(strides) == (2 if nq == 8 else 3), strides
    oidx = OracleIndex(oracle, dim, bits, rows_against(strides[:-1], n, dim, u, seed=5))
    q = queries_near(u, nq, dim, seed=6)
    ix = to_native(T, oidx)
    s, i = ix.search(q, k)
    assert ix.overflow_redos() == nq and ix.exact_redos() == 0
    os_, oi = oracle.search_fast(oidx.rot, oidx.seq, oidx.scales, q, k, bits, dim, n)
    assert np.array_equal(i, oi) and bits_equal(s, os_)
    ix.close()


# turbovec/src/lib.rs:22-52, tests/concurrent_search.rs: searches from many threads at once; here
# the waiting calls are merged into one launch, and every caller must get its own rows
@pytest.mark.parametrize("dev_buffers", [False, True])
def test_merged_calls_return_each_callers_rows(T, oracle, dev_buffers):
    torch = pytest.importorskip("torch")
    dim, n, k = 256, 20_011, 10
    oidx = OracleIndex(oracle, dim, 4, unit_gaussian(n, dim, seed=11))
    ix = to_native(T, oidx)
    n_threads, per_thread = 8, 12
    qs = [unit_gaussian(1 + (t % 3), dim, seed=100 + t) for t in range(n_threads)]     # 1 to 3 queries per call
    want = [oidx.search(q, k) for q in qs]
    mask = np.random.default_rng(12).random(n) < 0.3
    words = T.pack_mask(mask)[0]
    want_masked = [oidx.search(q, k, mask_words=words) for q in qs]
    bad = []
    dev_bufs = []
    if dev_buffers:                      # device buffers are made on this thread, before the callers start
        dev = torch.device("cuda:0")
        for q in qs:
            dev_bufs.append((torch.from_numpy(q).to(dev), torch.empty(len(q), k, device=dev),
                             torch.empty(len(q), k, dtype=torch.int64, device=dev)))
        torch.cuda.synchronize()

    def guarded(fn):
        def run(t):
            try:
                fn(t)
            except Exception as e:       # a thread's exception must fail the test, not vanish
                bad.append((t, repr(e)))
        return run

    def host_worker(t):
        for it in range(per_thread):
            masked = (t + it) % 4 == 0                      # some calls with another mask: never merged with the rest
            s, i = ix.search(qs[t], k, mask_words=words if masked else None)
            ws, wi = (want_masked if masked else want)[t]
            if not (np.array_equal(i, wi) and bits_equal(s, ws)):
                bad.append((t, it))

    def dev_worker(t):
        dq, ds, di = dev_bufs[t]
        for it in range(per_thread):
            ix.search_dev(dq.data_ptr(), len(qs[t]), k, ds.data_ptr(), di.data_ptr())
            if not (np.array_equal(di.cpu().numpy(), want[t][1]) and bits_equal(ds.cpu().numpy(), want[t][0])):
                bad.append((t, it))

    threads = [threading.Thread(target=guarded(dev_worker if dev_buffers else host_worker), args=(t,))
               for t in range(n_threads)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not bad, bad
    assert ix.merged_calls() > 0, "no two calls ever met: nothing was merged"
    ix.close()


def test_calls_of_several_chunks(T, oracle):
    """4096 + 77 queries in one call (the reference's Python sends 4096-row calls,
    turbovec-python/python/turbovec/__init__.py:18): five chunks enqueued back to back, their
    overflow flags read once; every row equals the same query searched in a small call."""
    dim, n, k = 256, 9_001, 10
    oidx = OracleIndex(oracle, dim, 4, unit_gaussian(n, dim, seed=21))
    ix = to_native(T, oidx)
    q = unit_gaussian(4096 + 77, dim, seed=22)
    s, i = ix.search(q, k)
    os_, oi = oracle.search_fast(oidx.rot, oidx.seq, oidx.scales, q, k, 4, dim, n)
    assert np.array_equal(i, oi) and bits_equal(s, os_)
    s2, i2 = ix.search(q[4090:4100], k)
    assert np.array_equal(i2, i[4090:4100]) and bits_equal(s2, s[4090:4100])
    ix.close()


def test_several_chunks_with_overflow_in_some(T, oracle):
    """Chunks of one call overflow independently: queries near the poisoned direction (chunk 1 of
    3) take the repeated pass, the Gaussian ones around them do not, all rows equal the oracle."""
    dim, n, k = 128, 60_000, 10
    rng = np.random.default_rng(31)
    u = rng.standard_normal(dim).astype(np.float32)
    u /= np.linalg.norm(u)
    strides, _ = ladder_for(T, dim, 4, n, 1024, k)
    oidx = OracleIndex(oracle, dim, 4, rows_against(strides[:-1], n, dim, u, seed=32))
    q = unit_gaussian(2048 + 300, dim, seed=33)
    q[1024 + 100: 1024 + 400] = queries_near(u, 300, dim, seed=34)
    ix = to_native(T, oidx)
    s, i = ix.search(q, k)
    assert ix.overflow_redos() >= 300 and ix.exact_redos() == 0
    os_, oi = oracle.search_fast(oidx.rot, oidx.seq, oidx.scales, q, k, 4, dim, n)
    assert np.array_equal(i, oi) and bits_equal(s, os_)
    ix.close()


# The reference refuses non-finite and huge query values before the seam (lib.rs:1374-1380).  A
# caller that skipped tv_validate_queries must still get the call back: any status, any rows for
# the bad queries, the good rows of the batch untouched, no hang.
@pytest.mark.parametrize("dim,nq", [(256, 5), (256, 64), (1536, 140), (128, 200)])
@pytest.mark.timeout(60)
def test_unvalidated_queries_return(T, oracle, dim, nq):
    n, k = 6_007, 10
    oidx = OracleIndex(oracle, dim, 4, unit_gaussian(n, dim, seed=41))
    ix = to_native(T, oidx)
    q = unit_gaussian(nq, dim, seed=42)
    want_s, want_i = ix.search(q, k)
    poison = {0: np.nan, 1: np.inf, 2: -np.inf, 3: 1e30, 4: -3e38}
    for row, val in poison.items():
        qq = q.copy()
        qq[row, row] = val
        if row == 3:
            qq[row] *= np.float32(1e30)
        try:
            s, i = ix.search(qq, k)
        except T.TurbovecHipError:
            continue
        good = np.arange(nq) != row
        assert np.array_equal(i[good], want_i[good]) and bits_equal(s[good], want_s[good]), val
    qq = np.full((nq, dim), np.nan, np.float32)              # every query bad at once
    try:
        ix.search(qq, k)
    except T.TurbovecHipError:
        pass
    s, i = ix.search(q, k)                                   # and the index still answers
    assert np.array_equal(i, want_i) and bits_equal(s, want_s)
    ix.set_score_mode(T.SCORE_L_U32)                         # the LUT scans, single and batched
    want_s, want_i = ix.search(q, k)
    for val in (np.nan, np.inf, 1e38):
        qq = q.copy()
        qq[1, 3] = val
        try:
            s, i = ix.search(qq, k)
        except T.TurbovecHipError:
            continue
        good = np.arange(nq) != 1
        assert np.array_equal(i[good], want_i[good]) and bits_equal(s[good], want_s[good]), val
    ix.close()


@pytest.mark.parametrize("nq", [4, 130])
def test_clustered_insertion_order_switches_to_the_row_level_ladder(T, nq):
    """A clustered corpus inserted cluster by cluster, queries next to stored rows: a query's few
    thousand near neighbours fill a run of consecutive blocks, of which the floorless first level
    (one row per block) sees two or three, so its floor is far too low and the queries overflow.
    The answer is still exact (the repeated pass), and the index then keeps to the ladder of
    row-level samples, on which the same searches do not overflow."""
    torch = pytest.importorskip("torch")
    dev = torch.device("cuda:0")
    dim, n, per_cluster, k = 768, 120_000, 4_000, 10
    gen = torch.Generator(device=dev)
    gen.manual_seed(3)
    centres = torch.randn(n // per_cluster, dim, device=dev, generator=gen)
    cid = torch.arange(n, device=dev) // per_cluster
    v = centres[cid] + 0.3 * torch.randn(n, dim, device=dev, generator=gen)
    ix = T.NativeIndex(dim, 4)
    torch.cuda.synchronize()
    ix.add_dev(v.data_ptr(), n)
    q = (v[:: n // nq][:nq] + 0.05 * torch.randn(nq, dim, device=dev, generator=gen)).cpu().numpy()
    before = ix.sampling_plan(nq, k)[0].tolist()           # the floorless level and the full scan
    assert len(before) == 2
    s, i = ix.search(q, k)
    first = ix.overflow_redos()
    assert first * 8 >= nq, "the layout did not overflow the floorless level often enough: the test tests nothing"
    assert ix.sampling_plan(nq, k)[0].tolist() != before   # switched to row-level samples (a sparser first level)
    for _ in range(3):
        s2, i2 = ix.search(q, k)
        assert np.array_equal(i2, i) and bits_equal(s2, s)
    assert ix.overflow_redos() == first and ix.exact_redos() == 0
    ix.set_path(1)                                         # the exact path
    s3, i3 = ix.search(q, k)
    ix.set_path(0)
    assert np.array_equal(i3, i) and bits_equal(s3, s)
    ix.close()
