"""The C-ABI library loads and exports every symbol include/nextdoor_amd.h declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "nextdoor_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nd_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_reference_surface():
    names = declared_symbols()
    for needed in ("nd_graph_load", "nd_sampler_set_graph", "nd_sampler_alloc", "nd_sampler_do_transit_parallel",
                   "nd_sampler_get_final_samples", "nd_sampler_final_sample_size", "nd_sampler_free_device",
                   "nd_init_sampling", "nd_sample", "nd_final_sample_length", "nd_final_samples_array",
                   "nd_free_device_memory"):
        assert needed in names


def test_library_exports_every_declared_symbol():
    from nextdoor_amd import _capi
    from nextdoor_amd.build import LIB_PATH
    assert os.path.exists(LIB_PATH), "build the library first: python -m nextdoor_amd.build"
    handle = ctypes.CDLL(LIB_PATH)
    for name in declared_symbols():
        assert hasattr(handle, name), name
    # the Python binding covers the same set
    assert sorted(_capi.SIGNATURES) == declared_symbols()


def test_app_registry_lists_the_reference_apps():
    import nextdoor_amd
    names = nextdoor_amd.app_names()
    for app in ("UniformRandomWalk", "DeepWalk", "PPR", "Node2Vec", "KHop", "WeightedNode2Vec"):
        assert app in names


def test_unknown_app_is_an_error_not_an_abort():
    import nextdoor_amd
    import pytest
    g = nextdoor_amd.Graph.from_edges([0, 1], [1, 0])
    with pytest.raises(nextdoor_amd.NextDoorError):
        nextdoor_amd.Sampler("NoSuchApp", g)


def test_bad_arguments_are_refused_before_anything_reaches_a_device():
    import numpy as np
    import nextdoor_amd
    import pytest
    g = nextdoor_amd.Graph.from_edges([0, 1, 2], [1, 2, 0])
    # a transit that is neither a vertex nor a "no vertex" value
    with pytest.raises(nextdoor_amd.NextDoorError, match="not a vertex"):
        nextdoor_amd.collective_neighborhood(g, np.array([[0, 7]], np.int32), 2, invalid=3, capacity=16)
    # room for fewer entries than the neighbourhoods hold
    with pytest.raises(nextdoor_amd.NextDoorError, match="capacity"):
        nextdoor_amd.collective_neighborhood(g, np.array([[0, 1]], np.int32), 2, invalid=3, capacity=1)
    # row offsets that run backwards, a column outside the graph
    with pytest.raises(nextdoor_amd.NextDoorError, match="monotone"):
        nextdoor_amd.Graph.from_csr([0, 2, 1, 3], [1, 2, 0])
    with pytest.raises(nextdoor_amd.NextDoorError, match="out of range"):
        nextdoor_amd.Graph.from_csr([0, 1, 2, 3], [1, 2, 9])


def test_app_registration_refuses_what_it_cannot_run():
    """nd_register_app, the door for apps built outside the library: another engine layout, a
    name that is taken and missing arguments are refused with a message; a good registration
    shows up in the list (its factory is never called here: no sampler is made)."""
    import ctypes as C
    import nextdoor_amd
    from nextdoor_amd import _capi
    L = _capi.lib()
    maker_type = C.CFUNCTYPE(C.c_void_p, C.c_char_p)
    maker = maker_type(lambda name: None)
    keep_alive.append(maker)
    fn = C.cast(maker, C.c_void_p)
    # the library's value: ND_ENGINE_ABI of include/nextdoor_amd.h in the upper half, struct sizes below
    abi = L.nd_engine_abi()
    text = open(os.path.join(ROOT, "include", "nextdoor_amd.h")).read()
    assert re.search(r"#define\s+ND_ENGINE_ABI\s+%d\b" % (abi >> 16), text)
    assert L.nd_register_app(b"HostSideProbeApp", fn, abi >> 16) == -2  # the bare version number is not enough
    assert L.nd_register_app(b"HostSideProbeApp", fn, abi + 1) == -2
    assert b"engine ABI" in L.nd_last_error()
    assert L.nd_register_app(b"KHop", fn, abi) == -3
    assert b"already registered" in L.nd_last_error()
    assert L.nd_register_app(None, fn, abi) != 0 and L.nd_register_app(b"HostSideProbeApp", None, abi) != 0
    assert "HostSideProbeApp" not in nextdoor_amd.app_names()
    assert L.nd_register_app(b"HostSideProbeApp", fn, abi) == 0
    assert "HostSideProbeApp" in nextdoor_amd.app_names()
    assert L.nd_register_app(b"HostSideProbeApp", fn, abi) == -3


keep_alive = []  # ctypes callbacks handed to the library must outlive the test


def test_an_app_whose_factory_gives_nothing_is_an_error():
    import nextdoor_amd
    import pytest
    if "HostSideProbeApp" not in nextdoor_amd.app_names():
        test_app_registration_refuses_what_it_cannot_run()
    g = nextdoor_amd.Graph.from_edges([0, 1], [1, 0])
    with pytest.raises(nextdoor_amd.NextDoorError, match="returned no engine"):
        nextdoor_amd.Sampler("HostSideProbeApp", g)


def test_the_sort_that_allocates_nothing_refuses_bad_calls_before_it_touches_a_device():
    """nd_sort_pairs_noalloc checks its arguments on the host first: too many pairs, and any
    overlap between the arrays of a call (equal pointers, an output inside an input's range,
    the two outputs inside each other), are refused with a message.  The addresses below are
    never dereferenced: every call here is refused before a HIP call is made."""
    import nextdoor_amd as nd
    L = nd._capi.lib()
    base = 1 << 40
    n = 1000

    def call(keys, vals, n_pairs, keys_out, vals_out):
        return L.nd_sort_pairs_noalloc(keys, vals, n_pairs, 20, keys_out, vals_out, None), L.nd_last_error().decode()

    rc, why = call(base, None, nd.SORT_PAIRS_NOALLOC_MAX + 1, base + (1 << 30), base + (2 << 30))
    assert rc == -2 and "at most" in why
    far = [base + i * (1 << 20) for i in range(4)]
    for keys, vals, keys_out, vals_out in [
            (far[0], far[1], far[0], far[3]),              # keys sorted in place
            (far[0], far[1], far[2], far[1]),              # values sorted in place
            (far[0], far[1], far[2], far[2]),              # both outputs one array
            (far[0], far[1], far[2], far[2] + 4 * n - 4),  # the outputs share their last / first word
            (far[0], far[1], far[0] + 4 * (n - 1), far[3]),  # an output starts inside an input
            (far[0], far[1], far[1] - 4, far[3]),          # an output ends inside an input
    ]:
        rc, why = call(keys, vals, n, keys_out, vals_out)
        assert rc == -3 and "overlap" in why, (keys, vals, keys_out, vals_out, rc, why)
    assert call(None, None, 0, None, None)[0] == 0  # nothing to sort
    assert call(None, None, 5, far[2], far[3])[0] != 0  # no input
