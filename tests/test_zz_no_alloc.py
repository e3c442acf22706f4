"""tv_search_dev_noalloc -- the search on the library's fixed scratch array, for callers that
cannot allocate device memory -- against tv_search_dev on the same device buffers: slots and
float scores bit for bit, on consecutive calls of shrinking size (the array keeps the previous
call's bytes), through the sampled path, its exact fallback and the all-queries-per-pass kernel;
and the refusal of a search that would not fit."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def T():
    from turbovec_amd import _lib
    _lib.lib()
    return _lib


def build(T, n, dim, bits, seed, duplicate_rows=False):
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    ix = T.NativeIndex(dim, bits)
    v = torch.randn(n, dim, device=dev, generator=gen)
    if duplicate_rows:
        v[:] = v[0]
    torch.cuda.synchronize()
    ix.add_dev(v.data_ptr(), n)
    return ix, gen


def both(ix, q, k, mask=None, n_allowed=0):
    """(scores, slots) of tv_search_dev and of tv_search_dev_noalloc for the same device buffers."""
    nq = q.shape[0]
    out = []
    for fn in (ix.search_dev, ix.search_dev_noalloc):
        s = torch.full((nq, k), float("nan"), device=q.device)
        i = torch.full((nq, k), -1, dtype=torch.int64, device=q.device)
        torch.cuda.synchronize()
        k_eff = fn(q.data_ptr(), nq, k, s.data_ptr(), i.data_ptr(),
                   None if mask is None else mask.data_ptr(), n_allowed)
        torch.cuda.synchronize()
        out.append((k_eff, s.cpu().numpy().ravel()[: nq * k_eff].view(np.uint32).copy(),
                    i.cpu().numpy().ravel()[: nq * k_eff].copy()))
    return out


def assert_same(pair):
    (ka, sa, ia), (kb, sb, ib) = pair
    assert ka == kb
    assert np.array_equal(ia, ib)
    assert np.array_equal(sa, sb)
    assert (ia >= 0).all()


@pytest.mark.parametrize("dim,bits,n", [(256, 4, 200_003), (128, 2, 150_001), (1536, 4, 40_000)])
def test_noalloc_equals_search_dev_on_consecutive_shrinking_calls(T, dim, bits, n):
    ix, gen = build(T, n, dim, bits, seed=dim + bits)
    dev = torch.device("cuda:0")
    q = torch.randn(160, dim, device=dev, generator=gen)
    rng = np.random.default_rng(3)
    m = rng.random(n) < 0.3
    words, allowed = T.pack_mask(m)
    d_words = torch.from_numpy(words.view(np.int64)).to(dev)
    # larger call first, smaller ones after it: 160 queries (wide kernel at 1536 dimensions,
    # tile groups elsewhere), then 33, then 5 with a mask, then 1
    assert_same(both(ix, q, 10))
    assert_same(both(ix, q[:33].contiguous(), 10))
    assert_same(both(ix, q[:5].contiguous(), 100, d_words, allowed))
    assert_same(both(ix, q[:1].contiguous(), 10))
    assert_same(both(ix, q[:7].contiguous(), 32, d_words, allowed))
    assert ix.overflow_redos() == 0
    ix.close()


def test_noalloc_exact_fallback_runs_inside_the_scratch(T):
    """Identical rows tie everywhere: the candidate segments overflow and the queries are redone
    through the exact lists, which must come out of the same fixed array."""
    ix, gen = build(T, 60_000, 64, 4, seed=9, duplicate_rows=True)
    q = torch.randn(6, 64, device="cuda:0", generator=gen)
    before = ix.overflow_redos()
    pair = both(ix, q, 10)
    assert_same(pair)
    assert np.array_equal(pair[1][2].reshape(6, 10), np.tile(np.arange(10), (6, 1)))
    assert ix.overflow_redos() >= before + 12       # both entry points took the fallback
    assert_same(both(ix, q[:2].contiguous(), 3))
    ix.close()


def test_noalloc_refuses_what_does_not_fit(T):
    ix, gen = build(T, 5_000, 1536, 4, seed=11)
    dev = torch.device("cuda:0")
    q = torch.randn(1024, 1536, device=dev, generator=gen)
    s = torch.zeros(1024, 10, device=dev)
    i = torch.zeros(1024, 10, dtype=torch.int64, device=dev)
    torch.cuda.synchronize()
    with pytest.raises(T.TurbovecHipError) as err:
        ix.search_dev_noalloc(q.data_ptr(), 1024, 10, s.data_ptr(), i.data_ptr())
    assert err.value.status == T.ERR_BAD_ARGUMENT
    assert "scratch" in str(err.value) and str(T.lib().tv_noalloc_scratch_bytes()) in str(err.value)
    assert float(s.abs().sum()) == 0.0              # nothing was written
    # the same index still answers through both entry points afterwards
    assert_same(both(ix, q[:64].contiguous(), 10))
    # degenerate calls: k = 0 and no queries write nothing and succeed
    assert ix.search_dev_noalloc(q.data_ptr(), 4, 0, s.data_ptr(), i.data_ptr()) == 0
    assert ix.search_dev_noalloc(q.data_ptr(), 0, 10, s.data_ptr(), i.data_ptr()) == 10
    ix.close()


def test_noalloc_takes_no_device_memory(T):
    """Free device memory and the index's own workspace stay what they were across calls of the
    entry point, on an index whose regular workspace was never sized for these searches."""
    ix, gen = build(T, 120_000, 256, 4, seed=13)
    dev = torch.device("cuda:0")
    q = torch.randn(96, 256, device=dev, generator=gen)
    s = torch.zeros(96, 10, device=dev)
    i = torch.zeros(96, 10, dtype=torch.int64, device=dev)
    torch.cuda.synchronize()
    ws0 = ix.workspace_bytes()
    free0 = torch.cuda.mem_get_info()[0]
    for nq in (96, 40, 1, 96):
        ix.search_dev_noalloc(q.data_ptr(), nq, 10, s.data_ptr(), i.data_ptr())
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    assert ix.workspace_bytes() == ws0
    ix.search_dev(q.data_ptr(), 96, 10, s.data_ptr(), i.data_ptr())      # the regular entry point does grow it
    assert ix.workspace_bytes()[0] > ws0[0]
    ix.close()
