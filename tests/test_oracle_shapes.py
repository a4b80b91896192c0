"""Shape algebra of the oracle against closed forms and the values the reference prints."""


def test_walk_shapes_match_readme_transcript(oracle):
    # README.md:88-92: "Final Size of each sample: 100", "Maximum Neighbors Sampled at each step: 1"
    d = oracle.app_desc(oracle.UNIFORM_WALK, 100, 1)
    assert oracle.final_sample_size(d) == 100
    L = oracle.lib()
    assert all(L.ndo_step_size_at_step(d, k) == 1 for k in range(100))
    assert L.ndo_number_of_transits(d, 7) == 1
    assert L.ndo_sub_warp_size_at_step(d, 0) == 1


def test_khop_shapes(oracle):
    d = oracle.app_desc(oracle.KHOP, 2, [25, 10])
    L = oracle.lib()
    assert oracle.final_sample_size(d) == 25 + 250
    assert L.ndo_step_size_at_step(d, 0) == 25 and L.ndo_step_size_at_step(d, 1) == 250
    assert L.ndo_step_size_at_step(d, -1) == 0
    assert L.ndo_sub_warp_size_at_step(d, 0) == 32 and L.ndo_sub_warp_size_at_step(d, 1) == 16


def test_collective_shapes(oracle):
    d = oracle.app_desc(oracle.LAYER_LITERAL, 5, 64, initial_size=64)
    L = oracle.lib()
    assert oracle.final_sample_size(d) == 320
    assert L.ndo_step_size_at_step(d, 2) == 192
    assert L.ndo_number_of_transits(d, 3) == 64


def test_max_bits(oracle):
    L = oracle.lib()
    # INVALID_VERTEX = n_vertices must be representable
    assert L.ndo_max_bits(56944) == 16
    assert L.ndo_max_bits(1 << 22) == 23
    assert L.ndo_max_bits(1 << 21) == 22
    assert L.ndo_max_bits(1) == 1
    assert L.ndo_max_bits(255) == 8 and L.ndo_max_bits(256) == 9


def test_kernel_classes(oracle):
    L = oracle.lib()
    # utils.hpp:491-497: grid 256, block 32, sub-warp 8
    assert L.ndo_kernel_class(256, 1) == 1 and L.ndo_kernel_class(255, 1) == 2
    assert L.ndo_kernel_class(8, 32) == 1 and L.ndo_kernel_class(7, 32) == 2
    assert L.ndo_kernel_class(1, 16) == 3 and L.ndo_kernel_class(1, 4) == 4
    assert L.ndo_kernel_class(31, 1) == 3 and L.ndo_kernel_class(7, 1) == 4
