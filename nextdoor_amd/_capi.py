"""ctypes binding of the C ABI declared in include/nextdoor_amd.h."""
import ctypes as C
import os

from .build import LIB_PATH

_lib = None

c_i32p = C.POINTER(C.c_int32)
c_f32p = C.POINTER(C.c_float)
c_i64p = C.POINTER(C.c_int64)

# name -> (restype, argtypes); every symbol include/nextdoor_amd.h declares
SIGNATURES = {
    "nd_last_error": (C.c_char_p, []),
    "nd_num_apps": (C.c_int, []),
    "nd_app_name": (C.c_char_p, [C.c_int]),
    "nd_engine_abi": (C.c_int, []),
    "nd_register_app": (C.c_int, [C.c_char_p, C.c_void_p, C.c_int]),
    "nd_graph_load": (C.c_int, [C.c_char_p, C.c_char_p, C.c_char_p, C.POINTER(C.c_void_p)]),
    "nd_graph_from_edges": (C.c_int, [C.c_int32, C.c_int64, c_i32p, c_i32p, c_f32p, C.POINTER(C.c_void_p)]),
    "nd_graph_from_csr": (C.c_int, [C.c_int32, C.c_int64, c_i32p, c_i32p, c_f32p, C.POINTER(C.c_void_p)]),
    "nd_graph_rmat": (C.c_int, [C.c_int, C.c_int, C.c_double, C.c_double, C.c_double, C.c_uint64, C.c_int,
                                C.POINTER(C.c_void_p)]),
    "nd_graph_chung_lu": (C.c_int, [C.c_int32, C.c_int64, C.c_double, C.c_uint64, C.POINTER(C.c_void_p)]),
    "nd_graph_num_vertices": (C.c_int32, [C.c_void_p]),
    "nd_graph_num_edges": (C.c_int64, [C.c_void_p]),
    "nd_graph_row_ptr": (c_i32p, [C.c_void_p]),
    "nd_graph_col": (c_i32p, [C.c_void_p]),
    "nd_graph_weight": (c_f32p, [C.c_void_p]),
    "nd_graph_max_weight": (c_f32p, [C.c_void_p]),
    "nd_graph_free": (None, [C.c_void_p]),
    "nd_sampler_create": (C.c_int, [C.c_char_p, C.POINTER(C.c_void_p)]),
    "nd_sampler_set_graph": (C.c_int, [C.c_void_p, C.c_void_p]),
    "nd_sampler_alloc": (C.c_int, [C.c_void_p, C.c_uint64]),
    "nd_sampler_do_transit_parallel": (C.c_int, [C.c_void_p, C.c_int]),
    "nd_sampler_do_sample_parallel": (C.c_int, [C.c_void_p]),
    "nd_sampler_check_results": (C.c_int, [C.c_void_p, C.POINTER(C.c_int)]),
    "nd_check_sampled_vertices": (C.c_int, [C.c_void_p, C.c_int, c_i32p, C.c_int, C.c_int, C.c_int64, c_i32p, c_i32p,
                                            C.c_int32]),
    "nd_sampler_get_final_samples": (C.c_int, [C.c_void_p, C.POINTER(c_i32p), c_i64p]),
    "nd_sampler_final_sample_size": (C.c_int, [C.c_void_p]),
    "nd_sampler_num_samples": (C.c_int64, [C.c_void_p]),
    "nd_sampler_initial_contents": (C.c_int, [C.c_void_p, C.POINTER(c_i32p), c_i64p]),
    "nd_sampler_invalid_vertex": (C.c_int32, [C.c_void_p]),
    "nd_sampler_max_bits": (C.c_int, [C.c_void_p]),
    "nd_sampler_steps": (C.c_int, [C.c_void_p]),
    "nd_sampler_step_size": (C.c_int, [C.c_void_p, C.c_int]),
    "nd_sampler_initial_sample_size": (C.c_int, [C.c_void_p]),
    "nd_sampler_sampling_type": (C.c_int, [C.c_void_p]),
    "nd_sampler_sample_state_bytes": (C.c_int64, [C.c_void_p]),
    "nd_sampler_get_sample_states": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64]),
    "nd_sampler_set_inversion_period": (C.c_int, [C.c_void_p, C.c_int]),
    "nd_sampler_set_launch_graph": (C.c_int, [C.c_void_p, C.c_int]),
    "nd_sampler_set_profiling": (C.c_int, [C.c_void_p, C.c_int]),
    "nd_sampler_phase_times": (C.c_int, [C.c_void_p, c_f32p]),
    "nd_sampler_get_adjacency": (C.c_int, [C.c_void_p, C.POINTER(c_i32p), C.POINTER(c_i32p), c_i64p,
                                           C.POINTER(C.POINTER(C.c_uint32)), c_i64p]),
    "nd_sampler_distinct": (C.c_int, [C.c_void_p]),
    "nd_sampler_get_distinct_counts": (C.c_int, [C.c_void_p, C.POINTER(c_i32p), c_i64p]),
    "nd_sampler_counter": (C.c_int64, [C.c_void_p, C.c_int]),
    "nd_sampler_free_device": (None, [C.c_void_p]),
    "nd_sampler_destroy": (None, [C.c_void_p]),
    "nd_init_sampling": (C.c_int, [C.c_char_p, C.c_char_p, C.c_uint64]),
    "nd_init_sampling_from_csr": (C.c_int, [C.c_char_p, C.c_int32, C.c_int64, c_i32p, c_i32p, c_f32p, C.c_uint64]),
    "nd_sample": (C.c_int, []),
    "nd_final_sample_length": (C.c_int64, []),
    "nd_final_samples_array": (c_i32p, []),
    "nd_free_device_memory": (None, []),
    "nd_philox_fill_uniform": (C.c_int, [C.c_uint64, C.c_uint32, C.c_uint64, C.c_int64, C.c_int, c_f32p]),
    "nd_philox_fill_step": (C.c_int, [C.c_uint64, C.c_uint32, C.c_int, C.c_uint64, C.c_int64, C.c_int, c_f32p]),
    "nd_sort_pairs": (C.c_int, [c_i32p, c_i32p, C.c_int64, C.c_int, c_i32p, c_i32p]),
    "nd_sort_pairs_noalloc": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "nd_load_balancing_thresholds": (C.c_int, [c_i32p]),
    "nd_classify_runs": (C.c_int, [c_i32p, C.c_int64, c_i32p, C.c_int32, C.c_int, C.c_int, c_i32p, C.c_int64,
                                   c_i64p, C.POINTER(C.c_uint8), c_i64p]),
    "nd_collective_neighborhood": (C.c_int, [C.c_void_p, c_i32p, C.c_int64, C.c_int32, C.c_int32, c_i32p, c_i32p, c_i32p,
                                             c_f32p, C.c_int64, c_i32p]),
    "nd_measure_gather_rate": (C.c_int, [C.c_int64, C.POINTER(C.c_double)]),
    "nd_measure_gather_rate_shaped": (C.c_int, [C.c_int64, C.c_int, C.c_int, C.POINTER(C.c_double)]),
    "nd_unique_transits": (C.c_int, [c_i32p, C.c_int64, C.c_int32, c_i32p, c_i32p, c_i32p, c_i64p, c_i64p]),
}


class NextDoorError(RuntimeError):
    pass


def lib():
    """Loads the in-tree library; builds it first only if it has never been built."""
    global _lib
    if _lib is not None:
        return _lib
    path = os.environ.get("NEXTDOOR_AMD_LIB", LIB_PATH)  # an explicitly chosen build of the library
    if path == LIB_PATH and not os.path.exists(LIB_PATH):
        from .build import build
        build()
    handle = C.CDLL(path)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(handle, name)  # AttributeError here = the library lacks a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = handle
    return _lib


def check(rc):
    if rc != 0:
        raise NextDoorError(lib().nd_last_error().decode())
