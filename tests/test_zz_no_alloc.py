"""The dedup entry point that allocates nothing (krk_dedup_noalloc) against krk_dedup, through
the C ABI: same unique ids, inverse map and count, bit for bit, on two calls in a row that share
the library's fixed work space, the second with a smaller request."""
import numpy as np
import pytest

from util import zipf_ids

pytestmark = pytest.mark.gpu

# torch (the caller-made stream of the second test) is imported before the library binds the
# device: its HIP runtime then is the one both use
try:
    import torch
except ImportError:
    torch = None


@pytest.fixture(scope="module")
def gpu_api():
    from kraken_amd import api as a
    a.lib()
    return a


def _free_bytes(api):
    import ctypes as C
    free, total = C.c_size_t(), C.c_size_t()
    assert api.lib().krk_mem_info(C.byref(free), C.byref(total)) == 0
    return free.value


def _both(api, ids, stream=None, check_memory=False):
    n = ids.size
    d_ids = api.DeviceArray.from_host(ids)
    ref_uids, ref_inv, ref_u = api.dedup(d_ids)
    uids = api.DeviceArray(max(n, 1), np.uint64)
    inv = api.DeviceArray(max(n, 1), np.int64)
    count = api.DeviceArray.from_host(np.array([-7], np.int64))
    api.synchronize()
    before = _free_bytes(api)
    rc = api.dedup_noalloc(d_ids, uids, inv, count, n=n, stream=stream)
    assert rc == 0, api.lib().krk_last_error_string()
    api.synchronize()
    if check_memory:
        assert _free_bytes(api) == before, "the call that allocates nothing changed the device's free memory"
    u = int(count.to_host()[0])
    assert u == ref_u
    assert np.array_equal(uids.to_host()[:u], ref_uids.to_host()[:u])
    assert np.array_equal(inv.to_host()[:n], ref_inv.to_host()[:n])
    return u


def test_no_alloc_dedup_matches_dedup_twice_in_a_row(gpu_api):
    api = gpu_api
    rng = np.random.default_rng(11)
    big = zipf_ids(rng, 1.05, 10**6, 200_000)
    big[::1000] = np.uint64(0xFFFFFFFFFFFFFFFF)          # the id that equals the index's empty marker
    small = zipf_ids(rng, 1.3, 10**5, 3_001)
    u_big = _both(api, big)
    # reuses the work space the first call dirtied; the device's free memory does not move
    u_small = _both(api, small, check_memory=True)
    assert 0 < u_small < u_big
    assert _both(api, np.arange(17, dtype=np.uint64)) == 17
    # the limit is refused with a clear error, nothing is launched
    n_over = api.DEDUP_NOALLOC_MAX + 1
    d = api.DeviceArray(n_over, np.uint64)
    rc = api.dedup_noalloc(d, d, None, api.DeviceArray(1, np.int64), n=n_over)
    assert rc == api.E_CAPACITY
    assert b"at most" in api.lib().krk_last_error_string()
    # an empty request writes a zero count
    count = api.DeviceArray.from_host(np.array([5], np.int64))
    assert api.dedup_noalloc(d, d, None, count, n=0) == 0
    api.synchronize()
    assert int(count.to_host()[0]) == 0


def test_no_alloc_dedup_on_a_stream_the_caller_made(gpu_api):
    """The launches go to the stream the caller names (here one that torch created, at the default
    priority), behind what the caller enqueued there, and the device's free memory stays where it
    was."""
    if torch is None or not torch.cuda.is_available():
        pytest.skip("needs torch with a visible GPU for a stream of the caller's own")
    api = gpu_api
    rng = np.random.default_rng(12)
    stream = torch.cuda.Stream()
    for n in (50_000, 700):
        assert _both(api, zipf_ids(rng, 1.1, 10**5, n), stream=stream.cuda_stream, check_memory=True) > 0
    stream.synchronize()
