"""Element-wise kernels as a class (spoc_amd/csrc/host/map_fuse.cpp): which IR generate_source tags map_f32, and that
the tag never lands on a kernel outside the class.  No GPU needed."""
import pytest

from map_kernels import MAPS, near_misses

MARK = "// sarek-hip-specialise: "


@pytest.mark.parametrize("name", sorted(MAPS))
def test_maps_are_tagged_and_still_lower_to_the_same_text(hip, name):
    src = hip.generate_source(MAPS[name]())
    first, rest = src.split("\n", 1)
    assert first == MARK + "map_f32"
    assert "__global__ void sarek_kern(" in rest and "tid < n" in rest


def test_the_bench_kernels_keep_their_own_tags(hip):
    """Vector add, copy and the triad are maps too, but their hand kernels compute in the CPU backend's double
    arithmetic: they keep their tags."""
    from spoc_amd import reference_kernels as rk
    assert hip.generate_source(rk.vector_add()).startswith(MARK + "vector_add_f32")
    assert hip.generate_source(rk.vector_copy()).startswith(MARK + "vector_copy_f32")
    assert hip.generate_source(rk.stream_triad()).startswith(MARK + "stream_triad_f32")


@pytest.mark.parametrize("name,ir", near_misses(), ids=[n for n, _ in near_misses()])
def test_near_misses_are_left_alone(hip, name, ir):
    assert not hip.generate_source(ir).startswith(MARK), name
