"""Element-wise kernels as a class (spoc_amd/csrc/host/map_fuse.cpp): which IR generate_source tags map_f32, and that
the tag never lands on a kernel outside the class.  No GPU needed."""
import pytest

from map_kernels import MAPS, MAX_TREES, TREES, near_misses, tree_near_misses

MARK = "// sarek-hip-specialise: "


@pytest.mark.parametrize("name", sorted(MAPS))
def test_maps_are_tagged_and_still_lower_to_the_same_text(hip, name):
    src = hip.generate_source(MAPS[name]())
    first, rest = src.split("\n", 1)
    assert first == MARK + "map_f32"
    assert "__global__ void sarek_kern(" in rest and ("tid < n" in rest or "tid < q" in rest)


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


@pytest.mark.parametrize("name", sorted(TREES))
def test_tree_sums_with_an_expression_in_front_are_tagged(hip, name):
    assert hip.generate_source(TREES[name](), block=(256, 1, 1)).startswith(MARK + "tree_sum_map_f32\n")


def test_the_reference_trees_keep_their_tags(hip):
    from spoc_amd import reference_kernels as rk
    assert hip.generate_source(rk.tree(False), block=(256, 1, 1)).startswith(MARK + "reduce_sum_block256_f32")
    assert hip.generate_source(rk.tree(True), block=(256, 1, 1)).startswith(MARK + "dot_block256_f32")


@pytest.mark.parametrize("name,ir", tree_near_misses(), ids=[n for n, _ in tree_near_misses()])
def test_tree_near_misses_are_left_alone(hip, name, ir):
    assert not hip.generate_source(ir, block=(256, 1, 1)).startswith(MARK), name


@pytest.mark.parametrize("name", sorted(MAX_TREES))
def test_maximum_trees_with_an_expression_in_front_are_tagged(hip, name):
    ir = MAX_TREES[name]()
    assert hip.generate_source(ir, block=(256, 1, 1)).startswith(MARK + "tree_max_map_f32\n")
    # "greater or equal" is another tree (it would pick another of two equal-comparing values, -0 and +0 say)
    assert "(gt (var b" in ir
    assert not hip.generate_source(ir.replace("(gt (var b", "(ge (var b", 1), block=(256, 1, 1)).startswith(MARK)
    assert not hip.generate_source(ir.replace("(i32 32)", "(i32 16)", 1), block=(256, 1, 1)).startswith(MARK)


def _compiles_for_gfx950(tmp_path, name, text):
    """hipcc cross-compiles without a GPU: the rebuilt text must be a complete HIP program for the target."""
    import subprocess
    src = tmp_path / (name + ".hip")
    src.write_text("#include <hip/hip_runtime.h>\n" + text)       # what hiprtc provides without being asked
    res = subprocess.run(["/opt/rocm/bin/hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature",
                          "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-c", str(src), "-o", str(tmp_path / (name + ".o"))],
                         capture_output=True, text=True)
    errors = [line for line in res.stderr.splitlines() if "error" in line and "packed-fp32-ops" not in line]
    assert res.returncode == 0 and not errors, res.stderr[-2000:]


def test_every_rebuilt_text_compiles_for_the_target(hip, tmp_path):
    """What run_source would hand to hiprtc on the GPU box, compiled here: every map alone, with block sums and with
    block maxima, every tree sum and maximum."""
    for name in sorted(MAPS):
        for reduce, pad in ((0, 0), (1, 0), (2, 0xC0600000)):
            text = hip.rebuilt_source(MAPS[name](), reduce, pad)
            assert 'extern "C" __global__' in text and "sarek_map(" in text
            assert ("sarek_f_wave_sum" in text) == (reduce == 1) and ("0xc0600000u" in text) == (reduce == 2)
            _compiles_for_gfx950(tmp_path, f"{name}_{reduce}", text)
    for name, make in sorted({**TREES, **MAX_TREES}.items()):
        text = hip.rebuilt_source(make())
        assert "sarek_tree(" in text
        _compiles_for_gfx950(tmp_path, name, text)


def test_rebuilt_source_refuses_everything_else(hip):
    from spoc_amd import reference_kernels as rk
    for ir in (rk.stream_triad(), rk.tree(False), near_misses()[0][1], rk.histogram()):
        with pytest.raises(hip.SarekHipError) as err:
            hip.rebuilt_source(ir)
        assert err.value.status == hip.E_UNSUPPORTED
    with pytest.raises(hip.SarekHipError):
        hip.rebuilt_source(MAPS["scale"](), reduce=3)


def _map_with_lets(lets, value, tid_name="tid"):
    """out[tid] <- VALUE under the given (name, expression) lets, over x, scalars a and b, and n."""
    tid = f"(var {tid_name} 9 i32)"
    body = f"(assign (lelem out {tid}) {value})"
    for k, (name, e) in reversed(list(enumerate(lets))):
        body = f"(let (var {name} {20 + k} f32) {e} {body})"
    return ("(kernel sarek_kern (params (param (var x 1 (vec f32))) (param (var out 2 (vec f32))) (param (var a 3 f32)) "
            f"(param (var b 4 f32)) (param (var n 5 i32))) (locals) (body (let {tid} (intr (Std) global_thread_id) "
            f"(if (lt {tid} (var n 5 i32)) {body}))) (native_fn true))")


def test_lets_that_take_a_name_again_in_a_map(hip, tmp_path):
    """A let may reuse a let's name or a scalar parameter's: the element function then holds the lowering's renamed
    variables.  A let that would hide the element's index, a vector, or one of the rebuilt text's own names keeps the
    kernel with the generated code."""
    xi, a = "(read x (var tid 9 i32))", "(var a 3 f32)"
    ir = _map_with_lets([("t", f"(mul {xi} {a})"), ("t", f"(add (var t 20 f32) {xi})"), ("a", "(mul (var t 21 f32) (var t 21 f32))")],
                        "(sub (var a 22 f32) (var b 4 f32))")
    assert hip.generate_source(ir).startswith(MARK + "map_f32\n")
    text = hip.rebuilt_source(ir, 1, 0)
    assert ("  float t = (x__e * a);\n  float t_2 = (t + x__e);\n  float a_2 = (t_2 * t_2);\n"
            "  sarek_f_res = (a_2 - b);\n") in text
    _compiles_for_gfx950(tmp_path, "rebound", text)
    for lets, value, tid_name in (
            ([("tid", "(f32 1.0)")], xi, "tid"),                       # out[tid] would mean another element
            ([("x", "(f32 1.0)")], "(var x 20 f32)", "tid"),           # hides the input vector
            ([("out", "(f32 1.0)")], xi, "tid"),                       # hides the output vector
            ([("x__e", "(f32 1.0)")], f"(add {xi} (var x__e 20 f32))", "tid"),
            ([("sarek_f_res", "(f32 1.0)")], xi, "tid"),
            ([], "(read x (var x__e 9 i32))", "x__e")):
        assert not hip.generate_source(_map_with_lets(lets, value, tid_name)).startswith(MARK), lets
