"""The entry point that allocates nothing (nd_sort_pairs_noalloc: device arrays in, device
arrays out, working memory in a fixed array inside the library) against the allocating entry
point it is a variant of (nd_sort_pairs), bit for bit, through the C ABI."""
import ctypes as C

import numpy as np
import pytest

import nextdoor_amd as nd

pytestmark = pytest.mark.gpu


class Hip:
    """Device memory and a stream straight from the HIP runtime the library itself runs on
    (the test needs nothing else from it; the arrays it hands over are the caller's)."""

    def __init__(self):
        nd.app_names()  # loads the library, and with it the HIP runtime it is linked against
        self.rt = C.CDLL("libamdhip64.so.7")
        for name in ("hipMalloc", "hipFree", "hipMemcpy", "hipMemset", "hipStreamCreate", "hipStreamDestroy",
                     "hipStreamSynchronize", "hipDeviceSynchronize"):
            getattr(self.rt, name).restype = C.c_int
        self.rt.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        self.rt.hipFree.argtypes = [C.c_void_p]
        self.rt.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        self.rt.hipMemset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        self.rt.hipStreamCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.rt.hipStreamDestroy.argtypes = [C.c_void_p]
        self.rt.hipStreamSynchronize.argtypes = [C.c_void_p]

    def ok(self, rc):
        assert rc == 0, f"HIP error {rc}"

    def malloc(self, nbytes):
        p = C.c_void_p()
        self.ok(self.rt.hipMalloc(C.byref(p), max(nbytes, 4)))
        return p.value

    def upload(self, arr):
        p = self.malloc(arr.nbytes)
        self.ok(self.rt.hipMemcpy(p, arr.ctypes.data, arr.nbytes, 1))  # hipMemcpyHostToDevice
        return p

    def download(self, p, n, dtype):
        out = np.empty(n, dtype=dtype)
        self.ok(self.rt.hipMemcpy(out.ctypes.data, p, out.nbytes, 2))  # hipMemcpyDeviceToHost
        return out

    def free(self, *ptrs):
        for p in ptrs:
            if p:
                self.ok(self.rt.hipFree(p))


@pytest.fixture(scope="module")
def hip():
    return Hip()


def sort_without_allocating(hip, keys, vals, key_bits):
    """Device arrays in and out, on a stream of the caller's."""
    n = len(keys)
    d_keys = hip.upload(keys)
    d_vals = 0 if vals is None else hip.upload(vals)
    d_keys_out, d_vals_out = hip.malloc(4 * n), hip.malloc(4 * n)
    # outputs start from a pattern no result can hold, so stale or unwritten entries show
    hip.ok(hip.rt.hipMemset(d_keys_out, 0xF9, 4 * n))
    hip.ok(hip.rt.hipMemset(d_vals_out, 0xF9, 4 * n))
    hip.ok(hip.rt.hipDeviceSynchronize())
    stream = C.c_void_p()
    hip.ok(hip.rt.hipStreamCreate(C.byref(stream)))
    try:
        nd.sort_pairs_noalloc(d_keys, d_vals, n, key_bits, d_keys_out, d_vals_out, stream.value)
        hip.ok(hip.rt.hipStreamSynchronize(stream))
        return hip.download(d_keys_out, n, np.int32), hip.download(d_vals_out, n, np.int32)
    finally:
        hip.ok(hip.rt.hipStreamDestroy(stream))
        hip.free(d_keys, d_vals, d_keys_out, d_vals_out)


def test_sort_without_allocation_matches_the_allocating_sort_twice_in_a_row(hip):
    rng = np.random.default_rng(7)
    # a large call first, then smaller ones: the library's working array still holds the first
    # call's contents; key widths with one, two, three and four digit passes (the passes
    # alternate between the output arrays and the working array, ending in the output arrays)
    cases = [(nd.SORT_PAIRS_NOALLOC_MAX, 23, True), (300001, 23, True), (4097, 9, False), (70000, 16, True),
             (2048, 1, True), (1, 8, False), (999, 32, True), (nd.SORT_PAIRS_NOALLOC_MAX, 8, False)]
    for n, bits, with_vals in cases:
        print("no-alloc sort n", n, "bits", bits, "values", with_vals, flush=True)
        keys = rng.integers(0, 1 << min(bits, 31), n, dtype=np.int64).astype(np.int32)
        vals = rng.integers(0, 1 << 31, n, dtype=np.int64).astype(np.int32) if with_vals else None
        want_k, want_v = nd.sort_pairs(keys, vals, bits)
        got_k, got_v = sort_without_allocating(hip, keys, vals, bits)
        assert np.array_equal(got_k, want_k), (n, bits)
        assert np.array_equal(got_v, want_v), (n, bits)
        # and both are the stable sort by the low `bits` bits
        order = np.argsort(keys.astype(np.int64) & ((1 << bits) - 1), kind="stable")
        assert np.array_equal(got_k, keys[order])
        assert np.array_equal(got_v, (np.arange(n, dtype=np.int32) if vals is None else vals)[order])


def test_sizes_beyond_the_working_array_are_refused(hip):
    n = nd.SORT_PAIRS_NOALLOC_MAX + 1
    a, b, c = hip.malloc(4 * n), hip.malloc(4 * n), hip.malloc(4 * n)
    try:
        with pytest.raises(nd.NextDoorError, match="at most"):
            nd.sort_pairs_noalloc(a, 0, n, 20, b, c)
        with pytest.raises(nd.NextDoorError, match="in place"):
            nd.sort_pairs_noalloc(a, 0, 16, 20, a, c)
        nd.sort_pairs_noalloc(0, 0, 0, 20, 0, 0)  # nothing to sort: no error, nothing touched
    finally:
        hip.free(a, b, c)
