"""IR -> HIP lowering and hot-kernel recognition (host logic; no GPU needed).

Golden parity: for the reference's benchmark kernels the HIP text must equal the text the
reference's own lowering produces for CUDA-dialect targets, which its CI keeps in
benchmarks/descriptions/generated/*_generated.md (fixtures: tests/golden/generated/).
Unit cases mirror sarek-cuda/test/test_sarek_ir_cuda.ml:27-251 with HIP spellings.
"""
import ctypes as C
import glob
import os

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
IR_DIR = os.path.join(HERE, "golden", "ir")
GEN_DIR = os.path.join(HERE, "golden", "generated")
MARK = "// sarek-hip-specialise: "

KERNELS = sorted(os.path.basename(p)[:-3] for p in glob.glob(os.path.join(IR_DIR, "*.ir")))
EXPECTED_TAGS = {
    "matrix_mul_tiled": "matmul_tiled_f32", "stream_triad": "stream_triad_f32",
    "reduction": "reduce_sum_block256_f32", "dot_product": "dot_block256_f32",
    "vector_add": "vector_add_f32", "vector_copy": "vector_copy_f32", "matrix_mul": "matmul_naive_f32",
    "transpose_naive": "transpose_naive_f32", "transpose_tiled": "transpose_tiled_f32",
    "radix_sort_histogram": "radix_histogram_i32", "radix_sort_scatter": "radix_scatter_i32",
    "reduction_max": "reduce_max_block256_f32:ff800000",
}


def split_tag(src):
    if src.startswith(MARK):
        first, rest = src.split("\n", 1)
        return first[len(MARK):], rest
    return "", src


def kernel_with_body(body, params=""):
    return f"(kernel sarek_kern (params {params}) (locals) (body {body}) (native_fn true))"


def body_text(hip, stmt, params=""):
    """Lowered text of one statement, without the kernel wrapper."""
    src = hip.generate_source(kernel_with_body(stmt, params))
    tag, src = split_tag(src)
    start = src.index(") {\n") + 4
    end = src.rindex("}\n}\n")
    return src[start:end]


def expr_text(hip, expr):
    out = body_text(hip, f"(expr {expr})")
    assert out.startswith("  ") and out.endswith(";\n")
    return out[2:-2]


def test_fixture_list():
    assert set(EXPECTED_TAGS) <= set(KERNELS) and len(KERNELS) == 15


@pytest.mark.parametrize("name", KERNELS)
def test_lowering_reproduces_golden_text(hip, name):
    ir = open(os.path.join(IR_DIR, name + ".ir")).read()
    expected = open(os.path.join(GEN_DIR, name + ".cuda.txt")).read()
    tag, src = split_tag(hip.generate_source(ir, block=(256, 1, 1)))
    assert src == expected
    assert tag == EXPECTED_TAGS.get(name, "")


def test_literals(hip):
    assert expr_text(hip, "(i32 42)") == "42"
    assert expr_text(hip, "(i64 42)") == "42LL"
    assert "." in expr_text(hip, "(f64 3.14)")
    assert expr_text(hip, "(bool true)") == "1"
    assert expr_text(hip, "(bool false)") == "0"
    assert expr_text(hip, "(f32 0.0)") == "0.0f"
    assert expr_text(hip, "(f32 2.5)") == "2.5f"
    assert expr_text(hip, "(f32 0.1)") == "0.10000000000000001f"   # "%.17g" + f
    assert expr_text(hip, "(f32 1e30)") == "1e+30f"
    # what "%.17g" prints as inf / nan (no C: the reference's text for such a constant does not compile) is written
    # with builtins, which the run-time compiler knows without a header
    assert expr_text(hip, "(f32 inf)") == "__builtin_inff()" and expr_text(hip, "(f64 -inf)") == "(-__builtin_inf())"
    assert expr_text(hip, "(f32 nan)") == '__builtin_nanf("")' and expr_text(hip, "(f64 nan)") == '__builtin_nan("")'
    # a whole-valued double keeps a decimal point: `2` is an int in C, (1 / 2) the integer division, -0 the integer 0
    assert expr_text(hip, "(f64 2.0)") == "2.0" and expr_text(hip, "(f64 -0.0)") == "-0.0"
    assert expr_text(hip, "(div (f64 1.0) (f64 2.0))") == "(1.0 / 2.0)" and expr_text(hip, "(f64 1e22)") == "1e+22"
    # the least int32 / int64 have no literal of their own type
    assert expr_text(hip, "(i32 -2147483648)") == "(-2147483647 - 1)"
    assert expr_text(hip, "(i32 -2147483647)") == "-2147483647"
    assert expr_text(hip, "(i64 -9223372036854775808)") == "(-9223372036854775807LL - 1)"
    assert expr_text(hip, "(i64 9223372036854775807)") == "9223372036854775807LL"


def test_operations(hip):
    assert expr_text(hip, "(var x 1 i32)") == "x"
    assert expr_text(hip, "(add (i32 1) (i32 2))") == "(1 + 2)"
    assert expr_text(hip, "(mul (var x 1 i32) (i32 3))") == "(x * 3)"
    assert expr_text(hip, "(neg (var x 1 i32))") == "(-x)"
    assert expr_text(hip, "(neg (neg (var x 1 i32)))") == "(-(-x))"
    # the minus of a negation and the minus of a negative literal never meet ("--3.5f" decrements a literal)
    assert expr_text(hip, "(neg (f32 -3.5))") == "(- -3.5f)"
    assert expr_text(hip, "(neg (i32 -5))") == "(- -5)"
    assert expr_text(hip, "(sub (var x 1 i32) (i32 -5))") == "(x - -5)"
    assert expr_text(hip, "(shl (var x 1 i32) (i32 2))") == "(x << 2)"
    assert expr_text(hip, "(if (lt (var x 1 i32) (i32 0)) (i32 1) (i32 2))") == "((x < 0) ? 1 : 2)"
    assert expr_text(hip, "(cast f32 (var x 1 i32))") == "(float)x"
    assert expr_text(hip, "(len v)") == "sarek_v_length"
    assert expr_text(hip, "(read v (var x 1 i32))") == "v[x]"


def test_statements(hip):
    assert body_text(hip, "(empty)") == ""
    assert body_text(hip, "(seq (empty) (empty))") == ""
    out = body_text(hip, "(assign (lvar (var result 1 i32 mut)) (i32 42))")
    assert out == "  result = 42;\n"
    out = body_text(hip, "(if (bool true) (empty))")
    assert out == "  if (1) {\n  }\n"
    out = body_text(hip, "(if (bool true) (empty) (empty))")
    assert "} else {" in out
    out = body_text(hip, "(while (lt (var i 1 i32) (i32 10)) (empty))")
    assert out.startswith("  while ((i < 10)) {")
    up = body_text(hip, "(for (var i 1 i32 mut) (i32 0) (i32 9) upto (empty))")
    assert up == "  for (int i = 0; i <= 9; i++) {\n  }\n"          # inclusive bound
    down = body_text(hip, "(for (var i 1 i32 mut) (i32 9) (i32 0) downto (empty))")
    assert down == "  for (int i = 9; i >= 0; i--) {\n  }\n"
    assert body_text(hip, "(let (var x 1 i32) (i32 42) (empty))") == "  int x = 42;\n"
    assert "double y = 3.14" in body_text(hip, "(letmut (var y 1 f64 mut) (f64 3.14) (empty))")
    # a let of type unit declares nothing (`void u = ...;` is no C): the value is evaluated for what it does
    assert body_text(hip, "(let (var u 1 unit) (unit) (assign (lvar (var r 2 i32 mut)) (i32 1)))") == "  (void)0;\n  r = 1;\n"
    assert body_text(hip, "(block (empty))") == "  {\n  }\n"
    assert body_text(hip, "(pragma (unroll) (empty))") == "  #pragma unroll\n"
    assert body_text(hip, '(native "asm volatile(\\"\\");")') == '  asm volatile("");\n'


def test_barriers_use_hip_spellings(hip):
    assert body_text(hip, "(barrier)") == "  __syncthreads();\n"
    assert body_text(hip, "(memfence)") == "  __threadfence();\n"
    warp = body_text(hip, "(warpbarrier)")
    assert "__syncwarp" not in warp and "__builtin_amdgcn_wave_barrier()" in warp


def test_intrinsics(hip):
    assert expr_text(hip, "(intr (Gpu) thread_idx_x)") == "threadIdx.x"
    assert expr_text(hip, "(intr (Gpu) block_dim_y)") == "blockDim.y"
    assert expr_text(hip, "(intr (Std) global_thread_id)") == "(threadIdx.x + blockIdx.x * blockDim.x)"
    assert expr_text(hip, "(intr (Std) global_size)") == "(blockDim.x * gridDim.x)"
    assert expr_text(hip, "(intr (Float32) sqrt (var x 1 f32))") == "sqrt(x)"
    assert expr_text(hip, "(intr (Float32) of_int (var x 1 i32))") == "(float)(x)"
    assert expr_text(hip, "(intr (Float32) add (var x 1 f32) (var y 2 f32))") == "(x + y)"
    # template resolved by the caller's registry wins over the built-in table
    assert expr_text(hip, '(intr (My) twice (template "(2 * %s)") (var x 1 i32))') == "(2 * x)"
    assert expr_text(hip, '(intr (My) f (template "my_f") (var x 1 i32) (i32 1))') == "my_f(x, 1)"
    assert expr_text(hip, "(intr (Mod Sub) unknown_fn (i32 1))") == "Mod.Sub.unknown_fn(1)"
    assert expr_text(hip, "(intr (Gpu) atomic_add (read h (i32 0)) (i32 1))") == "atomicAdd(&h[0], 1)"
    assert expr_text(hip, "(intr (Gpu) atomic_add (var h 1 (vec i32)) (i32 3) (i32 1))") == "atomicAdd(&h[3], 1)"
    # Stdlib.Int32 / Int64 by name (sarek/Sarek_stdlib/Int32.ml:30-88, Int64.ml:31-88)
    assert expr_text(hip, "(intr (Int32) abs (var a 1 i32))") == "abs(a)"
    assert expr_text(hip, "(intr (Int64) abs (var a 1 i64))") == "llabs(a)"
    assert expr_text(hip, "(intr (Sarek_stdlib Int32) logxor (var a 1 i32) (i32 3))") == "(a ^ 3)"
    assert expr_text(hip, "(intr (Int32) min (var a 1 i32) (i32 3))") == "min(a, 3)"
    # the rest of the standard library by name (Sarek_float64/Float64.ml:133-146, Math.ml:19-35, Gpu.ml:117-247)
    assert expr_text(hip, "(intr (Float64) of_int32 (var a 1 i32))") == "(double)(a)"
    assert expr_text(hip, "(intr (Float64) to_float32 (var d 1 f64))") == "(float)(d)"
    assert expr_text(hip, "(intr (Math) xor (var a 1 i32) (i32 3))") == "(a ^ 3)"
    assert expr_text(hip, "(intr (Gpu) spoc_powint (var a 1 i32) (i32 3))") == "spoc_powint(a, 3)"
    assert expr_text(hip, '(intr (Gpu) float64_of_int (template "(double)") (var a 1 i32))') == "(double)(a)"
    # the registry's templates are format strings (applied with Printf there, Sarek_ir_cuda.ml:360-396): %% is a %
    assert expr_text(hip, '(intr (Int32) mod_int32 (template "(%s %% %s)") (var a 1 i32) (i32 3))') == "(a % 3)"
    # a minus in a template keeps a space from an operand that begins with one
    assert expr_text(hip, '(intr (Int32) neg (template "(-%s)") (i32 -5))') == "(- -5)"
    # the logical shifts' templates leave an unsigned value: OCaml's result is signed again
    assert expr_text(hip, "(intr (Int32) shift_right_logical (var a 1 i32) (i32 3))") == "(int)((unsigned int)a >> 3)"
    assert expr_text(hip, '(intr (Int64) shift_right_logical (template "((unsigned long)%s >> %s)") (var a 1 i64) (i32 3))') \
        == "(long long)((unsigned long)a >> 3)"


def test_vector_params_get_length_arguments(hip):
    src = hip.generate_source(kernel_with_body(
        "(empty)", "(param (var v 1 (vec f64))) (param (var k 2 i64)) (param (var flag 3 bool))"))
    assert "__global__ void sarek_kern(double* __restrict__ v, int sarek_v_length, long long k, int flag) {" in src
    assert src.startswith('\nextern "C" {\n') and src.endswith("}\n}\n")


def test_records_variants_and_helpers(hip):
    ir = """
    (kernel k (params (param (var ps 1 (vec (record Geo.point (x f32) (y f32))))))
      (locals (shared tile f32 (i32 64)) (local (var acc 2 f32 mut) (f32 0.0)))
      (body (match (var s 3 (variant shape (Circle f32) (Rect f32 f32) (Empty)))
              (case (Circle r) (assign (lvar (var acc 2 f32 mut)) (var r 4 f32)))
              (case (Rect w h) (assign (lvar (var acc 2 f32 mut)) (mul (var w 5 f32) (var h 6 f32))))
              (case _ (empty))))
      (types (Geo.point (x f32) (y f32)))
      (variants (shape (Circle f32) (Rect f32 f32) (Empty)))
      (funcs (func sq (params (var a 7 f32)) f32 (return (mul (var a 7 f32) (var a 7 f32)))))
      (native_fn false))"""
    src = hip.generate_source(ir)
    assert "enum { Circle = 0, Rect = 1, Empty = 2 };" in src
    assert "typedef struct {\n  int tag;\n  union {\n    float Circle_v;\n    struct { float _0; float _1; } Rect_v;\n  } data;\n} shape;" in src
    assert "__device__ __host__ inline shape make_shape_Rect(float v0, float v1) {" in src
    assert "typedef struct {\n  float x;\n  float y;\n} Geo_point;" in src
    assert "__device__ float sq(float a) {\n  return (a * a);\n}" in src
    assert "Geo_point* __restrict__ ps, int sarek_ps_length" in src
    assert "  __shared__ float tile[64];\n  float acc = 0.0f;\n" in src
    assert "switch (s.tag) {" in src and "case Circle: {" in src and "float r = s.data.Circle_v;" in src
    assert "float w = s.data.Rect_v._0;" in src and "default: {" in src


@pytest.mark.parametrize("text,needle", [
    ("(kernel k (params) (locals) (body (frobnicate)))", "unknown statement form"),
    ("(kernel k (params) (locals) (body (empty))", "unbalanced"),
    ("(kernel k (params) (locals))", "without a (body"),
    ("(kernel k (params (param (var x 1 q8))) (locals) (body (empty)))", "unknown type"),
])
def test_parse_errors(hip, text, needle):
    with pytest.raises(hip.SarekHipError) as e:
        hip.generate_source(text)
    assert e.value.status == hip.E_PARSE and needle in e.value.message


def test_codegen_error_for_array_creation_outside_let(hip):
    with pytest.raises(hip.SarekHipError) as e:
        hip.generate_source(kernel_with_body("(expr (newarray f32 (i32 4) shared))"))
    assert e.value.status == hip.E_CODEGEN


def test_output_buffer_protocol(hip):
    ir = open(os.path.join(IR_DIR, "stream_triad.ir")).read().encode()
    needed = C.c_size_t(0)
    rc = hip.lib.sarek_hip_generate_source(ir, None, None, 0, C.byref(needed))
    assert rc == hip.E_BUFFER_TOO_SMALL and needed.value > 100
    buf = C.create_string_buffer(needed.value)
    assert hip.lib.sarek_hip_generate_source(ir, None, buf, len(buf), C.byref(needed)) == 0
    assert buf.value.decode().startswith(MARK + "stream_triad_f32\n")


# ---- recognition is strict: near misses are NOT taken over --------------------------

def triad_ir(expr):
    return kernel_with_body(
        "(let (var tid 6 i32) (intr (Std) global_thread_id) (if (lt (var tid 6 i32) (var n 5 i32)) "
        f"(assign (lelem a (var tid 6 i32)) {expr})))",
        "(param (var a 1 (vec f32))) (param (var b 2 (vec f32))) (param (var c 3 (vec f32))) "
        "(param (var scalar 4 f32)) (param (var n 5 i32))")


B, Cc, S = "(read b (var tid 6 i32))", "(read c (var tid 6 i32))", "(var scalar 4 f32)"


@pytest.mark.parametrize("expr,tag", [
    (f"(add {B} (mul {Cc} {S}))", "stream_triad_f32"),
    (f"(add (mul {S} {Cc}) {B})", "stream_triad_f32"),            # commuted operands: same value
    # other element-wise kernels: not the triad's hand kernel (the CPU backend's double arithmetic), but the class
    # of maps that is rebuilt from its own expression
    (f"(add {Cc} (mul {B} {S}))", "map_f32"),                      # b and c swapped: different kernel
    (f"(sub {B} (mul {Cc} {S}))", "map_f32"),
    (f"(add {B} (mul {Cc} (f32 3.0)))", "map_f32"),
    (f"(add {B} (mul (read c (add (var tid 6 i32) (i32 1))) {S}))", ""),
])
def test_triad_recognition_is_exact(hip, expr, tag):
    assert split_tag(hip.generate_source(triad_ir(expr)))[0] == tag


def test_recognition_survives_renaming_and_nesting(hip):
    ir = open(os.path.join(IR_DIR, "matrix_mul_tiled.ir")).read()
    renamed = (ir.replace("tile_a", "sh_one").replace("tile_b", "sh_two").replace("sum", "accum")
               .replace("(block ", "(seq ").replace("thread_idx_", "thread_id_"))
    assert split_tag(hip.generate_source(renamed))[0] == "matmul_tiled_f32"


def test_tiled_matmul_near_misses_fall_back(hip):
    ir = open(os.path.join(IR_DIR, "matrix_mul_tiled.ir")).read()
    assert split_tag(hip.generate_source(ir.replace("(i32 16)", "(i32 8)")))[0] == ""
    # a barrier removed: no longer the same program
    assert split_tag(hip.generate_source(ir.replace("(barrier)", "(empty)", 1)))[0] == ""
    # transposed B access
    swapped = ir.replace("(read b (add (mul (var b_row", "(read b (add (mul (var col", 1)
    assert split_tag(hip.generate_source(swapped))[0] == ""


def test_reduction_with_other_operator_is_not_taken(hip):
    ir = open(os.path.join(IR_DIR, "reduction.ir")).read()
    assert split_tag(hip.generate_source(ir.replace("(add (read sdata", "(mul (read sdata", 1)))[0] == ""
    assert split_tag(hip.generate_source(ir.replace("(i32 64)", "(i32 65)", 1)))[0] == ""


def test_data_movement_and_naive_matmul_near_misses_fall_back(hip):
    def tag_of(name, old=None, new=None):
        ir = open(os.path.join(IR_DIR, name + ".ir")).read()
        if old is not None:
            assert old in ir
            ir = ir.replace(old, new, 1)
        return split_tag(hip.generate_source(ir))[0]
    assert tag_of("vector_add") == "vector_add_f32"
    assert tag_of("vector_add", "(add (read a", "(sub (read a") == "map_f32"      # a map, but not the vector add
    assert tag_of("vector_add", "(lt (var tid 5 i32) (var n 4 i32))", "(le (var tid 5 i32) (var n 4 i32))") == ""
    assert tag_of("vector_copy", "(read a (var tid 4 i32))", "(read a (i32 0))") == ""
    # row and column swapped in the store: another matrix
    assert tag_of("matrix_mul", "(lelem c (add (mul (var row 8 i32) (var n 5 i32)) (var col 9 i32)))",
                  "(lelem c (add (mul (var col 9 i32) (var n 5 i32)) (var row 8 i32)))") == ""
    assert tag_of("matrix_mul", "(sub (var k 6 i32) (i32 1))", "(var k 6 i32)") == ""     # one step too many
    # a "transpose" that does not transpose, and a tile pitch of 16 (same result, other program)
    assert tag_of("transpose_naive", "(add (mul (var col 7 i32) (var height 4 i32)) (var row 8 i32))",
                  "(add (mul (var row 8 i32) (var width 3 i32)) (var col 7 i32))") == ""
    assert tag_of("transpose_tiled", "(i32 17)", "(i32 16)") == ""
    assert tag_of("transpose_tiled", "(lt (var write_col 15 i32) (var height 4 i32))",
                  "(lt (var write_col 15 i32) (var width 3 i32))") == ""


def test_histogram_recognition_and_near_misses(hip):
    from spoc_amd import reference_kernels
    hist = reference_kernels.histogram()
    assert split_tag(hip.generate_source(hist))[0] == "histogram_i32"
    # `()` and the empty statement are the same nothing
    assert split_tag(hip.generate_source(hist.replace("(expr (unit))", "(empty)")))[0] == "histogram_i32"
    assert split_tag(hip.generate_source(hist.replace("(i32 256)", "(i32 128)")))[0] == ""       # smaller block histogram
    assert split_tag(hip.generate_source(hist.replace("(mod (read input", "(div (read input")))[0] == ""
    assert split_tag(hip.generate_source(hist.replace("(i32 1))", "(i32 2))", 1)))[0] == ""       # counts by two
    assert split_tag(hip.generate_source(hist.replace("(barrier)", "(empty)", 1)))[0] == ""
    radix = open(os.path.join(IR_DIR, "radix_sort_histogram.ir")).read()
    assert split_tag(hip.generate_source(radix.replace("(shr ", "(shl ")))[0] == ""
    assert split_tag(hip.generate_source(radix.replace("(read local_hist (var tid 7 i32)))", "(i32 1))", 1)))[0] == ""


def test_radix_scatter_near_misses_fall_back(hip):
    ir = open(os.path.join(IR_DIR, "radix_sort_scatter.ir")).read()
    assert split_tag(hip.generate_source(ir))[0] == "radix_scatter_i32"
    assert split_tag(hip.generate_source(ir.replace("(i32 1))", "(i32 2))", 1)))[0] == ""            # every other slot
    assert split_tag(hip.generate_source(ir.replace("(lelem output (var pos 10 i32))", "(lelem output (var gid 7 i32))")))[0] == ""
    assert split_tag(hip.generate_source(ir.replace("(var counters 3 (vec i32)) (var digit 9 i32)",
                                                    "(var counters 3 (vec i32)) (i32 0)")))[0] == ""
    assert split_tag(hip.generate_source(ir.replace("(assign (lelem output (var pos 10 i32)) (var value 8 i32))",
                                                    "(assign (lelem output (var pos 10 i32)) (var digit 9 i32))")))[0] == ""


def test_an_atomic_in_an_unused_binding_is_part_of_the_program(hip):
    """`let _old = atomic_add ... in` binds a value nobody reads, and still changes memory: a triad
    that also counts its calls is not the triad."""
    expr = f"(add {B} (mul {Cc} {S}))"
    counted = kernel_with_body(
        "(let (var tid 6 i32) (intr (Std) global_thread_id) (if (lt (var tid 6 i32) (var n 5 i32)) "
        "(let (var _old 7 i32) (intr (Gpu) atomic_add_global_int32 (var hits 8 (vec i32)) (i32 0) (i32 1)) "
        f"(assign (lelem a (var tid 6 i32)) {expr}))))",
        "(param (var a 1 (vec f32))) (param (var b 2 (vec f32))) (param (var c 3 (vec f32))) "
        "(param (var scalar 4 f32)) (param (var n 5 i32)) (param (var hits 8 (vec i32)))")
    tag, src = split_tag(hip.generate_source(counted))
    assert tag == "" and "atomicAdd" in src
    # five parameters, the atomic on `a` reinterpreted is still an atomic: not taken either
    same_params = triad_ir(expr).replace(
        "(assign (lelem a", "(let (var _old 7 i32) (intr (Gpu) atomic_add_global_int32 (var a 1 (vec f32)) (i32 0) (i32 1)) "
        "(assign (lelem a", 1).replace(f"{expr})))", f"{expr}))))", 1)
    assert split_tag(hip.generate_source(triad_ir(expr)))[0] == "stream_triad_f32"
    assert split_tag(hip.generate_source(same_params))[0] == ""


def reduction_max_ir(pad="(f32 -1000000.0)"):
    """The kernel as benchmarks/bench_reduction_max.ml:18-100 writes it today (the golden
    text predates it and fills with Float.neg_infinity, a free variable)."""
    ir = open(os.path.join(IR_DIR, "reduction_max.ir")).read()
    free = "(var Float.neg_infinity"
    i = ir.index(free)
    j = ir.index(")", i) + 1
    return ir[:i] + pad + ir[j:]


def test_reduction_max_recognition_carries_the_fill_value(hip):
    import struct
    tag, src = split_tag(hip.generate_source(reduction_max_ir()))
    assert tag == "reduce_max_block256_f32:" + struct.pack(">f", -1000000.0).hex()
    assert "sdata[tid] = -1000000.0f;" in src
    assert split_tag(hip.generate_source(reduction_max_ir("(f32 -inf)")))[0] == "reduce_max_block256_f32:ff800000"
    # the golden form pads with OCaml's Float.neg_infinity by name (benchmarks/generate_backend_code.ml:164): minus
    # infinity; another free variable there is another program
    golden = open(os.path.join(IR_DIR, "reduction_max.ir")).read()
    assert split_tag(hip.generate_source(golden))[0] == "reduce_max_block256_f32:ff800000"
    assert "Float.neg_infinity" in golden
    assert split_tag(hip.generate_source(golden.replace("Float.neg_infinity", "Float.infinity")))[0] == ""
    # "<" instead of ">" is a min tree: another program
    assert split_tag(hip.generate_source(reduction_max_ir().replace("(gt ", "(lt ", 1)))[0] == ""
    assert split_tag(hip.generate_source(reduction_max_ir().replace("(i32 32)", "(i32 33)", 1)))[0] == ""


def test_nesting_depth_is_bounded(hip):
    """Every pass recurses over the tree; the reader refuses trees deep enough to endanger the
    caller's stack instead of crashing, and accepts anything a real kernel could hold."""
    def nested(d):
        return "(kernel k (params) (locals) (body " + "(seq " * d + "(empty)" + ")" * d + "))"
    assert "sarek_kern" not in hip.generate_source(nested(1900))
    for d in (2100, 200000):
        with pytest.raises(hip.SarekHipError, match="nesting deeper than 2000"):
            hip.generate_source(nested(d))
    lets = 1500
    ir = ("(kernel k (params (param (var o 1 (vec i32)))) (locals) (body " +
          "".join(f"(let (var x{i} {i + 2} i32) (add (i32 {i}) "
                  f"{('(var x%d %d i32)' % (i - 1, i + 1)) if i else '(i32 0)'}) " for i in range(lets)) +
          f"(assign (lelem o (i32 0)) (var x{lets - 1} {lets + 1} i32))" + ")" * lets + "))")
    assert f"int x{lets - 1} = " in hip.generate_source(ir)


def test_damaged_ir_is_refused_not_crashed_on(hip):
    """Seeded damage to the fixture kernels (atoms swapped for other atoms, pieces cut out, doubled
    or replaced, texts truncated): the reader and the lowering answer every one of them with a
    status, the ones that still mean something with a source."""
    import ctypes as C
    import random
    import re
    rng = random.Random(20240)
    texts = [open(os.path.join(IR_DIR, k + ".ir")).read() for k in KERNELS]
    spare = ["i32", "f32", "(var x 1 i32)", "add", "read", "let", "seq", "(i32 0)", "shared", "vec", "-",
             "999999999999999999999", '"', "template", "match", "case", "record", "variant", "app", "for", "upto", "mut"]
    seen = {}
    for it in range(1500):
        t = rng.choice(texts)
        if it % 2 == 0:
            toks = re.findall(r'\(|\)|"[^"]*"|[^\s()]+', t)
            atoms = [k for k, x in enumerate(toks) if x not in "()"]
            for _ in range(rng.randint(1, 4)):
                a, b = rng.choice(atoms), rng.choice(atoms)
                toks[a] = toks[b] if rng.random() < 0.7 else rng.choice(spare)
            t = " ".join(toks)
        else:
            for _ in range(rng.randint(1, 3)):
                if not t:
                    break
                i = rng.randrange(len(t))
                j = min(len(t), i + rng.randint(1, 40))
                kind = rng.randint(0, 4)
                t = (t[:i] + t[j:], t[:i] + t[i:j] * 2 + t[j:], t[:i] + rng.choice(spare) + t[j:],
                     t[:i] + rng.choice(spare) + t[i:], t[:i])[kind]
        buf, need = C.create_string_buffer(1 << 16), C.c_size_t(0)
        rc = hip.lib.sarek_hip_generate_source(t.encode(), None, buf, len(buf), C.byref(need))
        seen[rc] = seen.get(rc, 0) + 1
        if rc == hip.OK:
            assert b"__global__" in buf.value
        else:
            assert hip.lib.sarek_hip_last_error()
    assert set(seen) <= {hip.OK, hip.E_PARSE, hip.E_CODEGEN} and seen[hip.OK] > 20 and seen[hip.E_PARSE] > 500


def test_a_binding_that_reads_what_its_scope_changes_is_not_inlined(hip):
    """`let x = e in body` keeps x at the value e had when it was bound.  A recogniser that replaces
    x by e everywhere would take these kernels for the templates they resemble and serve them with
    a hand kernel that computes something else."""
    fixture = lambda name: open(os.path.join(IR_DIR, name)).read()     # noqa: E731
    # block sum whose stored value is the block's first element, read before the tree runs
    red = fixture("reduction.ir")
    assert split_tag(hip.generate_source(red))[0] == "reduce_sum_block256_f32"
    first_barrier = red.index("(barrier)") + len("(barrier)")
    hoisted = (red[:first_barrier] + "\n (let (var first 99 f32) (read sdata (i32 0)) (seq" + red[first_barrier:])
    hoisted = hoisted.replace("(assign (lelem output (intr (Gpu) block_idx_x)) (read sdata (i32 0)))",
                              "(assign (lelem output (intr (Gpu) block_idx_x)) (var first 99 f32))")
    hoisted = hoisted.replace("(barrier))))))\n (native_fn", "(barrier))))))))\n (native_fn")
    tag, src = split_tag(hip.generate_source(hoisted))
    assert tag == "" and "float first = sdata[0];" in src
    # the same binding placed after the tree reads the finished sum: the template's own program
    last = red.rindex("(block (if (eq")
    late = (red[:last] + "(let (var total 99 f32) (read sdata (i32 0)) (seq " +
            red[last:].replace("(read sdata (i32 0))", "(var total 99 f32)")
            .replace("(barrier))))))\n (native_fn", "(barrier))))))))\n (native_fn"))
    assert "float total = sdata[0];" in hip.generate_source(late)
    assert split_tag(hip.generate_source(late))[0] == ""      # a barrier follows in its scope: kept as written, no match, JIT

    # tiled matmul that stores the accumulator's value from before the loop
    mm = fixture("matrix_mul_tiled.ir")
    assert split_tag(hip.generate_source(mm))[0] == "matmul_tiled_f32"
    stale = mm.replace("(letmut (var sum 15 f32 mut) (f32 0.0)\n (seq",
                       "(letmut (var sum 15 f32 mut) (f32 0.0)\n (let (var s0 98 f32) (var sum 15 f32 mut) (seq", 1)
    stale = stale.replace("(var col 12 i32))) (var sum 15 f32 mut))))))))))))))\n (native_fn",
                          "(var col 12 i32))) (var s0 98 f32)))))))))))))))\n (native_fn", 1)
    tag, src = split_tag(hip.generate_source(stale))
    assert tag == "" and "float s0 = sum;" in src

    # a triad whose operand was read before an earlier store to the same vector (in place: a = a + c*s
    # with the old a[tid] saved, then a[tid] cleared, then the triad stored)
    saved = kernel_with_body(
        "(let (var tid 6 i32) (intr (Std) global_thread_id) (if (lt (var tid 6 i32) (var n 5 i32)) "
        "(let (var old 7 f32) (read b (var tid 6 i32)) (seq "
        "(assign (lelem b (var tid 6 i32)) (f32 0.0)) "
        f"(assign (lelem a (var tid 6 i32)) (add (var old 7 f32) (mul {Cc} {S})))))))",
        "(param (var a 1 (vec f32))) (param (var b 2 (vec f32))) (param (var c 3 (vec f32))) "
        "(param (var scalar 4 f32)) (param (var n 5 i32))")
    tag, src = split_tag(hip.generate_source(saved))
    assert tag == "" and "float old = b[tid];" in src
    # the same binding with nothing stored to b in its scope is the triad
    plain = saved.replace("(assign (lelem b (var tid 6 i32)) (f32 0.0)) ", "")
    assert split_tag(hip.generate_source(plain))[0] == "stream_triad_f32"


def test_recognition_does_not_depend_on_how_index_arithmetic_is_written(hip):
    """int32 +, -, * form a ring: bracketing, operand order, distribution and named or folded constants do not
    change an index, so they must not change what a kernel is recognised as.  (No IR printed by the reference's
    own front end is at hand: the fixtures were derived from its lowering rules, so the recogniser has to take
    every spelling of the same arithmetic.)"""
    mm = open(os.path.join(IR_DIR, "matrix_mul_tiled.ir")).read()
    tag = lambda ir: split_tag(hip.generate_source(ir))[0]                     # noqa: E731
    assert tag(mm) == "matmul_tiled_f32"
    ts = "(var tile_size 13 i32)"
    # the tile size written as a literal everywhere
    literal = mm.replace(ts, "(i32 16)").replace("(let (i32 16) (i32 16)", f"(let {ts} (i32 16)")
    assert literal.count(ts) == 1 and tag(literal) == "matmul_tiled_f32"
    # ceil(k / 16) with the constants folded, or bracketed the other way
    folded = mm.replace(f"(div (sub (add (var k 6 i32) {ts}) (i32 1)) {ts})", "(div (add (var k 6 i32) (i32 15)) (i32 16))")
    assert folded != mm and tag(folded) == "matmul_tiled_f32"
    other = mm.replace(f"(sub (add (var k 6 i32) {ts}) (i32 1))", f"(add (var k 6 i32) (sub {ts} (i32 1)))")
    assert other != mm and tag(other) == "matmul_tiled_f32"
    # operands the other way round, a product distributed
    swapped = mm.replace(f"(add (mul (var t 16 i32 mut) {ts}) (var tx 9 i32))", f"(add (var tx 9 i32) (mul {ts} (var t 16 i32 mut)))")
    assert swapped != mm and tag(swapped) == "matmul_tiled_f32"
    rowcol = mm.replace("(add (var ty 10 i32) (mul (intr (Gpu) block_dim_y) (intr (Gpu) block_idx_y)))",
                        "(add (mul (intr (Gpu) block_idx_y) (intr (Gpu) block_dim_y)) (var ty 10 i32))")
    assert rowcol != mm and tag(rowcol) == "matmul_tiled_f32"
    # the loop bound as num_tiles + (-1)
    bound = mm.replace("(sub (var num_tiles 14 i32) (i32 1))", "(add (var num_tiles 14 i32) (i32 -1))")
    assert bound != mm and tag(bound) == "matmul_tiled_f32"
    # ... and what is NOT the same arithmetic stays out
    assert tag(mm.replace(f"(div (sub (add (var k 6 i32) {ts}) (i32 1)) {ts})", f"(div (add (var k 6 i32) {ts}) {ts})")) == ""
    assert tag(mm.replace(f"(add (mul (var t 16 i32 mut) {ts}) (var tx 9 i32))", f"(add (mul (var t 16 i32 mut) {ts}) (var ty 10 i32))", 1)) == ""
    assert tag(mm.replace("(sub (var num_tiles 14 i32) (i32 1))", "(var num_tiles 14 i32)")) == ""
    # f32 arithmetic is not a ring: (b + c*s) re-bracketed with an extra term is another value (an element-wise
    # kernel still, but not the triad)
    assert tag(triad_ir(f"(add (add {B} (mul {Cc} {S})) (f32 0.0))")) == "map_f32"

    # thread index spelled out instead of the global_thread_id intrinsic, in either order
    tri = open(os.path.join(IR_DIR, "stream_triad.ir")).read()
    assert tag(tri) == "stream_triad_f32"
    spelled = tri.replace("(intr (Std) global_thread_id)",
                          "(add (mul (intr (Gpu) block_idx_x) (intr (Gpu) block_dim_x)) (intr (Gpu) thread_idx_x))")
    assert spelled != tri and tag(spelled) == "stream_triad_f32"
    red = open(os.path.join(IR_DIR, "reduction.ir")).read()
    short = red.replace("(add (intr (Gpu) thread_idx_x) (mul (intr (Gpu) block_dim_x) (intr (Gpu) block_idx_x)))",
                        "(intr (Std) global_thread_id)")
    assert short != red and tag(short) == "reduce_sum_block256_f32"
    # the tree's partner index tid + 64 written as 64 + tid
    assert tag(red.replace("(add (var tid 5 i32) (i32 64))", "(add (i32 64) (var tid 5 i32))")) == "reduce_sum_block256_f32"
    assert tag(red.replace("(add (var tid 5 i32) (i32 64))", "(add (i32 63) (var tid 5 i32))")) == ""


def test_stencil_and_box_filter_are_recognised_and_near_misses_are_not(hip):
    """A stencil with another divisor, or neighbours added in another association, is another program."""
    from spoc_amd import reference_kernels
    st, cv = reference_kernels.stencil_2d(), reference_kernels.conv2d()
    mark = "// sarek-hip-specialise: "
    assert hip.generate_source(st).startswith(mark + "stencil_2d_f32")
    assert hip.generate_source(cv).startswith(mark + "conv2d_f32")
    for text, old, new in [(st, "(f32 5.0)", "(f32 4.0)"), (cv, "(f32 9.0)", "(f32 8.0)"),
                           # (a + b is b + a bit for bit; (a + b) + c is not a + (b + c))
                           (st, "(add (add (var up 8 f32) (var down 9 f32)) (var left 10 f32))",
                            "(add (var up 8 f32) (add (var down 9 f32) (var left 10 f32)))"),
                           (st, "(var left 10 f32)) (var right 11 f32)) (var center 12 f32))",
                            "(var center 12 f32)) (var right 11 f32)) (var left 10 f32))"),
                           (cv, "(eq (var y 8 i32) (i32 0))", "(eq (var y 8 i32) (i32 1))")]:
        assert old in text
        assert not hip.generate_source(text.replace(old, new)).startswith(mark)


# ---- mutation tests of the recognisers: a kernel that differs from a template in one token is another program ----

_MUTATIONS = {"add": ["sub", "mul"], "sub": ["add"], "mul": ["add", "div"], "div": ["mul"], "mod": ["div"],
              "lt": ["le", "gt"], "le": ["lt"], "gt": ["ge", "lt"], "ge": ["gt"], "eq": ["ne"], "ne": ["eq"],
              "and": ["or"], "or": ["and"], "shl": ["shr"], "shr": ["shl"], "bitand": ["bitor"], "bitor": ["bitand"],
              "bitxor": ["bitor"]}


def _single_token_mutants(ir):
    """(position, mutant text) for every operator swapped for a neighbour, every int32 constant moved by one either
    way, every f32 constant moved by one, every loop turned round."""
    import re
    for m in re.finditer(r"\(([a-z_]+)\b|\((i32|f32) (-?[0-9.e+]+)\)|\b(upto)\b", ir):
        if m.group(1) in _MUTATIONS:
            for alt in _MUTATIONS[m.group(1)]:
                yield m.start(1), ir[:m.start(1)] + alt + ir[m.end(1):]
        elif m.group(2) == "i32":
            for d in (1, -1):
                yield m.start(3), ir[:m.start(3)] + str(int(m.group(3)) + d) + ir[m.end(3):]
        elif m.group(2) == "f32":
            yield m.start(3), ir[:m.start(3)] + repr(float(m.group(3)) + 1.0) + ir[m.end(3):]
        elif m.group(4):
            yield m.start(4), ir[:m.start(4)] + "downto" + ir[m.end(4):]


def _tag_or_none(hip, ir):
    try:
        return split_tag(hip.generate_source(ir, block=(256, 1, 1)))[0]
    except hip.SarekHipError:
        return None


@pytest.mark.parametrize("name", sorted(EXPECTED_TAGS))
def test_no_single_token_mutant_of_a_template_keeps_its_tag(hip, name):
    """The hand kernels stand in for fifteen exact programs.  Every operator of a recognised kernel swapped for a
    neighbour (+ for -, < for <=, ...), every integer constant moved by one, every float constant changed, every
    loop turned round gives a kernel that computes something else -- none of them may keep the template's tag."""
    ir = open(os.path.join(IR_DIR, name + ".ir")).read()
    tag = EXPECTED_TAGS[name]
    mutants = list(_single_token_mutants(ir))
    assert len(mutants) >= 2
    assert [m for _, m in mutants if _tag_or_none(hip, m) == tag] == []


def test_tree_class_mutants_keep_their_tag_only_inside_the_expression(hip):
    """The tree classes take any expression where the reference's tree reads its input (and any fill constant in the
    maximum tree); everything else is the tree to the letter.  A single-token mutant keeps the class tag exactly when
    the token lies in the expression or is the fill value."""
    import sys
    sys.path.insert(0, HERE)
    import map_kernels

    def span_after(ir, head, start=0):
        at = ir.index(head, start) + len(head)
        depth, i = 0, at
        while True:
            depth += {"(": 1, ")": -1}.get(ir[i], 0)
            i += 1
            if depth == 0:
                return at, i

    store = "(assign (lelem sdata (var tid 5 i32)) "
    for name, make in list(map_kernels.TREES.items()) + list(map_kernels.MAX_TREES.items()):
        ir = make()
        tag = _tag_or_none(hip, ir)
        assert tag in ("tree_sum_map_f32", "tree_max_map_f32"), name
        leaf = span_after(ir, store)
        fill = span_after(ir, store, leaf[1])          # the guard's else branch: the padding value
        kept = outside = 0
        for at, mutant in _single_token_mutants(ir):
            free = leaf[0] <= at < leaf[1] or (tag == "tree_max_map_f32" and fill[0] <= at < fill[1])
            same = _tag_or_none(hip, mutant) == tag
            if free:
                kept += same
            else:
                outside += 1
                assert not same, (name, ir[max(0, at - 60):at + 30])
        assert kept >= 1 and outside >= 40, (name, kept, outside)


def test_random_expressions_lower_to_text_the_device_compiler_takes(hip, tmp_path):
    """150 seeded integer kernels (arithmetic, bit operations, shifts, negations of negative literals, casts through
    float, `if` expressions, `not` / `and` / `or` in the guard) and 150 seeded float maps, lowered and handed to the
    device compiler's front end in one translation unit: the text must parse, whatever the operands of a unary
    minus or a cast begin with."""
    import random
    import shutil
    import subprocess
    import sys
    sys.path.insert(0, HERE)
    import map_kernels
    from spoc_amd import reference_kernels as rk
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc to parse the text with")

    def int_expr(rng, depth, leaves):
        if depth == 0:
            return rng.choice(leaves + [rk.i32(rng.randint(-9, 12))])
        a, b = int_expr(rng, depth - 1, leaves), int_expr(rng, depth - 1, leaves)
        pick = rng.randint(0, 7)
        if pick == 0:
            return rk.op(rng.choice(["add", "sub", "mul"]), a, b)
        if pick == 1:
            return rk.op(rng.choice(["bitand", "bitor", "bitxor"]), a, b)
        if pick == 2:
            return rk.op(rng.choice(["shl", "shr"]), a, rk.i32(rng.randint(0, 5)))
        if pick == 3:
            return f"(neg {a})"
        if pick == 4:
            return f"(bitnot {a})"
        if pick == 5:
            return f"(if {rk.op(rng.choice(['lt', 'le', 'gt', 'ge', 'eq', 'ne']), a, b)} {a} {b})"
        if pick == 6:
            return rk.op("mod", a, rk.add(rk.op("bitand", b, rk.i32(7)), rk.i32(1)))
        return f"(cast i32 (cast f32 {a}))"

    texts = ["#include <hip/hip_runtime.h>\n"]
    for seed in range(150):
        rng = random.Random(seed)
        rk.fresh()
        params = [("x", "(vec i32)"), ("out", "(vec i32)"), ("k", "i32"), ("n", "i32")]
        for p, t in params:
            rk.var(p, t)
        tid = rk.var("tid")
        value = int_expr(rng, rng.randint(2, 4), [tid, rk.var("k"), rk.read("x", tid)])
        guard = rng.choice([f"(not {rk.lt(tid, rk.var('k'))})",
                            f"(and {rk.lt(tid, rk.var('n'))} (or {rk.op('ge', tid, rk.i32(0))} {rk.op('ne', rk.var('k'), rk.i32(-2))}))"])
        body = rk.let(tid, rk.intr("global_thread_id", "Std"),
                      rk.if_(rk.lt(tid, rk.var("n")),
                             rk.if_(guard, rk.assign_elem("out", tid, value), rk.assign_elem("out", tid, f"(neg {rk.i32(-7)})"))))
        texts.append(hip.generate_source(rk.kernel(params, body)).replace("sarek_kern", f"ints_{seed}"))
        texts.append(hip.generate_source(map_kernels.random_map(1000 + seed)[0]).replace("sarek_kern", f"floats_{seed}"))
    path = tmp_path / "random_kernels.hip"
    path.write_text("\n".join(texts))
    done = subprocess.run([hipcc, "--offload-arch=gfx950", "--cuda-device-only", "-fsyntax-only", "-w", str(path)],
                          capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-3000:]


REBOUND = {
    # name: (body, the text it lowers to, what v holds after one thread has run it, from OCaml's scoping)
    "nested": ("(let (var x 1 i32) (i32 1) (let (var x 2 i32) (add (var x 1 i32) (i32 1)) "
               "(assign (lelem v (i32 0)) (var x 2 i32))))",
               "  int x = 1;\n  int x_2 = (x + 1);\n  v[0] = x_2;\n", {0: 2}),
    "siblings": ("(seq (let (var x 1 i32) (i32 1) (assign (lelem v (i32 0)) (var x 1 i32))) "
                 "(let (var x 2 i32) (i32 2) (assign (lelem v (i32 1)) (var x 2 i32))))",
                 "  int x = 1;\n  v[0] = x;\n  int x_2 = 2;\n  v[1] = x_2;\n", {0: 1, 1: 2}),
    "a parameter": ("(let (var n 5 i32) (add (var n 2 i32) (i32 1)) (assign (lelem v (i32 0)) (var n 5 i32)))",
                    "  int n_2 = (n + 1);\n  v[0] = n_2;\n", {0: 4}),
    "a loop counter": ("(let (var i 1 i32) (i32 2) (seq (for (var i 2 i32 mut) (i32 0) (var i 1 i32) upto "
                       "(assign (lelem v (var i 2 i32)) (add (var i 2 i32) (i32 10)))) "
                       "(assign (lelem v (i32 3)) (var i 1 i32))))",
                       "  int i = 2;\n  for (int i_2 = 0; i_2 <= i; i_2++) {\n    v[i_2] = (i_2 + 10);\n  }\n  v[3] = i;\n",
                       {0: 10, 1: 11, 2: 12, 3: 2}),
    "inside a branch": ("(let (var x 1 i32) (i32 1) (seq (if (bool true) (let (var x 2 i32) (mul (var x 1 i32) (i32 3)) "
                        "(assign (lelem v (i32 0)) (var x 2 i32)))) (assign (lelem v (i32 1)) (var x 1 i32))))",
                        "  int x = 1;\n  if (1) {\n    int x_2 = (x * 3);\n    v[0] = x_2;\n  }\n  v[1] = x;\n", {0: 3, 1: 1}),
    "three deep": ("(let (var x 1 i32) (i32 1) (let (var x 2 i32) (add (var x 1 i32) (i32 1)) (let (var x 3 i32) "
                   "(add (var x 2 i32) (i32 1)) (assign (lelem v (i32 0)) (var x 3 i32)))))",
                   "  int x = 1;\n  int x_2 = (x + 1);\n  int x_3 = (x_2 + 1);\n  v[0] = x_3;\n", {0: 3}),
    "a name already of that form": ("(let (var x_2 1 i32) (i32 5) (let (var x 2 i32) (i32 1) (let (var x 3 i32) "
                                    "(add (var x 2 i32) (var x_2 1 i32)) (assign (lelem v (i32 0)) (var x 3 i32)))))",
                                    "  int x_2 = 5;\n  int x = 1;\n  int x_3 = (x + x_2);\n  v[0] = x_3;\n", {0: 6}),
    # a let without a body in sequence with what follows is how a module's constant reaches the kernel
    # (Sarek_lower_ir.ml:634-671); the use's id says which binding it means
    "a constant named like a parameter": ("(seq (let (var n 7 i32) (i32 9) (empty)) (assign (lelem v (i32 0)) (var n 2 i32)))",
                                          "  int n_2 = 9;\n  v[0] = n;\n", {0: 3}),
    "two constants of one name": ("(seq (let (var s 7 i32) (i32 1) (empty)) (let (var s 8 i32) (i32 2) (empty)) "
                                  "(assign (lelem v (i32 0)) (var s 8 i32)))",
                                  "  int s = 1;\n  int s_2 = 2;\n  v[0] = s_2;\n", {0: 2}),
}
REBOUND_PARAMS = "(param (var v 1 (vec i32))) (param (var n 2 i32))"


@pytest.mark.parametrize("name", REBOUND)
def test_a_name_bound_again_gets_a_variable_of_its_own(hip, name):
    """OCaml lets a kernel bind a name again (`let x = 1 in let x = x + 1 in ...`), and the IR keeps the source's
    names (sarek/ppx/Sarek_lower_ir.ml:237 prints `v.var_name`).  Printed as they are, `int x = 1; int x = (x + 1);`
    is a redefinition in one C block and reads its own uninitialised self in a nested one, so the reference's text for
    such a kernel (Sarek_ir_cuda.ml:367-376, the same names) does not compile or computes something else.  Here the
    value is printed with the outer meaning and the new variable is called x_2, x_3, ... for the length of its body;
    a kernel that binds no name twice comes out as before (the golden texts above)."""
    body, text, _ = REBOUND[name]
    assert body_text(hip, body, REBOUND_PARAMS) == text


def test_rebound_names_in_helpers_and_match_cases(hip):
    ir = """
    (kernel k (params (param (var out 1 (vec f32))) (param (var r 2 f32)))
      (locals)
      (body (match (var s 3 (variant shape (Circle f32) (Rect f32 f32)))
              (case (Circle r) (assign (lelem out (i32 0)) (add (var r 4 f32) (var r 4 f32))))
              (case (Rect r h) (let (var h 7 f32) (mul (var r 5 f32) (var h 6 f32)) (assign (lelem out (i32 1)) (var h 7 f32))))))
      (variants (shape (Circle f32) (Rect f32 f32)))
      (funcs (func sq (params (var a 8 f32)) f32 (let (var a 9 f32) (mul (var a 8 f32) (var a 8 f32)) (return (var a 9 f32)))))
      (native_fn false))"""
    src = hip.generate_source(ir)
    assert "__device__ float sq(float a) {\n  float a_2 = (a * a);\n  return a_2;\n}" in src
    assert "float r_2 = s.data.Circle_v;" in src and "out[0] = (r_2 + r_2);" in src
    assert "float r_2 = s.data.Rect_v._0;" in src and "float h = s.data.Rect_v._1;" in src
    assert "float h_2 = (r_2 * h);" in src and "out[1] = h_2;" in src


def test_rebound_names_parse_as_device_code(hip, tmp_path):
    import shutil
    import subprocess
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc to parse the text with")
    texts = ["#include <hip/hip_runtime.h>\n"]
    for k, (body, _, _) in enumerate(REBOUND.values()):
        texts.append(hip.generate_source(kernel_with_body(body, REBOUND_PARAMS)).replace("sarek_kern", f"rebound_{k}"))
    path = tmp_path / "rebound.hip"
    path.write_text("\n".join(texts))
    done = subprocess.run([hipcc, "--offload-arch=gfx950", "--cuda-device-only", "-fsyntax-only", "-Wall", "-Werror=uninitialized",
                           "-Wno-unused-variable", str(path)], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-3000:]


def test_the_program_model_on_known_cases(hip):
    """The tests' walker of integer IR (ir_programs.evaluate) against the results the re-binding cases above fix by
    hand, and against loops whose bounds the body changes: OCaml evaluates a `for`'s bounds once."""
    import numpy as np
    import ir_programs
    for name, (body, _, want) in REBOUND.items():
        v = np.full(8, -1, np.int32)
        ir_programs.evaluate(kernel_with_body(body, REBOUND_PARAMS), {"v": v, "n": 3}, 1)
        expected = np.full(8, -1, np.int32)
        for at, value in want.items():
            expected[at] = value
        assert np.array_equal(v, expected), name
    for name, (body, _, want) in LOOP_BOUNDS.items():
        v = np.full(8, -1, np.int32)
        ir_programs.evaluate(kernel_with_body(body, REBOUND_PARAMS), {"v": v, "n": 3}, 1)
        assert v.tolist() == want, name


M = "(var m 7 i32 mut)"
LOOP_BOUNDS = {
    # name: (body, lowered text, v after one thread with n = 3)
    "a bound the body lowers": (
        f"(letmut {M} (i32 5) (for (var i 8 i32 mut) (i32 0) {M} upto (seq (assign (lelem v (var i 8 i32 mut)) {M}) "
        f"(assign (lvar {M}) (sub {M} (i32 1))))))",
        "  int m = 5;\n  for (int i = 0, sarek_to_i = m; i <= sarek_to_i; i++) {\n    v[i] = m;\n    m = (m - 1);\n  }\n",
        [5, 4, 3, 2, 1, 0, -1, -1]),
    "downwards, to an element the body overwrites": (
        "(seq (assign (lelem v (i32 7)) (i32 2)) (for (var i 8 i32 mut) (i32 5) (read v (i32 7)) downto "
        "(seq (assign (lelem v (var i 8 i32 mut)) (i32 9)) (assign (lelem v (i32 7)) (i32 4)))))",
        "  v[7] = 2;\n  for (int i = 5, sarek_to_i = v[7]; i >= sarek_to_i; i--) {\n    v[i] = 9;\n    v[7] = 4;\n  }\n",
        [-1, -1, 9, 9, 9, 9, -1, 4]),
    "fixed bounds stay in the condition": (
        "(let (var a 9 i32) (i32 2) (for (var i 8 i32 mut) (var a 9 i32) (add (var n 2 i32) (var a 9 i32)) upto "
        "(for (var j 10 i32 mut) (i32 0) (var i 8 i32 mut) upto (assign (lelem v (var j 10 i32 mut)) (var i 8 i32 mut)))))",
        "  int a = 2;\n  for (int i = a; i <= (n + a); i++) {\n    for (int j = 0; j <= i; j++) {\n      v[j] = i;\n    }\n  }\n",
        [5, 5, 5, 5, 5, 5, -1, -1]),
}


@pytest.mark.parametrize("name", LOOP_BOUNDS)
def test_a_loop_bound_the_body_may_change_is_evaluated_once(hip, name):
    """`for i = 0 to !m do ... m := !m - 1 done` runs to the value m had at the start in OCaml, on the Native backend
    and in the reference's IR walker (Sarek_ir_interp.ml:858-872: stop_val is computed before the loop); the
    reference's device text repeats the bound in the condition (Sarek_ir_cuda.ml:391-409), which evaluates it before
    every turn.  Here such a bound is kept in a variable of the statement's scope; a bound of constants, immutable
    variables, thread indices and loop counters is printed in the condition as before."""
    body, text, _ = LOOP_BOUNDS[name]
    assert body_text(hip, body, REBOUND_PARAMS) == text


def test_seeded_integer_programs_parse_as_device_code(hip, tmp_path):
    """120 seeded programs of lets, mutable variables, loops and branches whose names hide each other all the time
    (ir_programs.random_program), lowered and handed to the device compiler's front end: no redefinition, no use of
    a variable in its own initialiser."""
    import shutil
    import subprocess
    import ir_programs
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc to parse the text with")
    texts = ["#include <hip/hip_runtime.h>\n"]
    for seed in range(120):
        ir, _, _ = ir_programs.random_program(seed)
        text = hip.generate_source(ir).replace("sarek_kern", f"program_{seed}")
        texts.append(text.replace("helper0(", f"helper0_{seed}(").replace("helper1(", f"helper1_{seed}("))
    path = tmp_path / "programs.hip"
    path.write_text("\n".join(texts))
    done = subprocess.run([hipcc, "--offload-arch=gfx950", "--cuda-device-only", "-fsyntax-only", "-Wall",
                           "-Werror=uninitialized", "-Wno-unused-variable", "-Wno-unused-but-set-variable",
                           "-Wno-self-assign", "-Wno-tautological-compare", "-Wno-parentheses-equality", str(path)],
                          capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-3000:]


SHAPE = "(variant shape (Circle f32) (Rect f32 f32) (Empty))"
MATCH_AS_A_VALUE = f"""(kernel sarek_kern (params (param (var xs 1 (vec f32))) (param (var dst 2 (vec f32))) (param (var n 3 i32))) (locals)
 (body (let (var tid 4 i32) (intr (Std) global_thread_id) (if (lt (var tid 4 i32) (var n 3 i32))
   (let (var x 5 f32) (read xs (var tid 4 i32))
   (let (var s 6 {SHAPE}) (if (gt (var x 5 f32) (f32 1.0)) (variant shape Circle (var x 5 f32))
                             (if (lt (var x 5 f32) (f32 -1.0)) (variant shape Rect (var x 5 f32) (f32 2.0)) (variant shape Empty)))
     (assign (lelem dst (var tid 4 i32))
             (match (var s 6 {SHAPE}) (case (Circle x) (mul (var x 7 f32) (var x 7 f32)))
                                      (case (Rect w h) (mul (var w 8 f32) (var h 9 f32)))
                                      (case _ (var x 5 f32)))))))))
 (variants (shape (Circle f32) (Rect f32 f32) (Empty))) (native_fn true))"""


def test_a_match_used_as_a_value_binds_its_patterns(hip):
    """`dst.(tid) <- (match s with Circle x -> x *. x | Rect (w, h) -> w *. h | _ -> x)`: nested conditionals on the
    tag as the reference prints them (Sarek_ir_cuda.ml:179-208), with each case's variables standing for the payload
    they name -- the reference leaves them undeclared.  The Circle case's x hides the let's x inside that case only."""
    text = hip.generate_source(MATCH_AS_A_VALUE)
    assert ("dst[tid] = ((s.tag == Circle) ? (s.data.Circle_v * s.data.Circle_v) : "
            "((s.tag == Rect) ? (s.data.Rect_v._0 * s.data.Rect_v._1) : x));") in text


MATCH_WITH_A_VARIABLE_PATTERN = f"""(kernel sarek_kern (params (param (var xs 1 (vec f32))) (param (var dst 2 (vec f32))) (param (var n 3 i32))) (locals)
 (body (let (var tid 4 i32) (intr (Std) global_thread_id) (if (lt (var tid 4 i32) (var n 3 i32))
   (let (var x 5 f32) (read xs (var tid 4 i32))
   (let (var s 6 {SHAPE}) (if (gt (var x 5 f32) (f32 1.0)) (variant shape Circle (var x 5 f32)) (variant shape Rect (var x 5 f32) (f32 3.0)))
     (seq (match (var s 6 {SHAPE})
            (case (Circle r) (assign (lelem dst (var tid 4 i32)) (var r 7 f32)))
            (case (? other) (assign (lelem dst (var tid 4 i32))
                                    (match (var other 8 {SHAPE}) (case (Rect w h) (mul (var w 9 f32) (var h 10 f32)))
                                                                 (case (? rest) (f32 -1.0))))))))))))
 (variants (shape (Circle f32) (Rect f32 f32) (Empty))) (native_fn true))"""


def test_a_pattern_that_names_the_value(hip):
    """`| other -> ...`: the front end lowers a variable pattern to a constructor pattern with an empty name
    (Sarek_lower_ir.ml:556-559), for which the reference prints `case : {`.  Here it is the default case with the
    variable bound to the value matched, as a statement and -- the variable standing for the value -- as a value."""
    text = hip.generate_source(MATCH_WITH_A_VARIABLE_PATTERN)
    assert "      default: {\n        auto other = s;\n" in text
    assert "dst[tid] = ((other.tag == Rect) ? (other.data.Rect_v._0 * other.data.Rect_v._1) : -1.0f);" in text
    with pytest.raises(hip.SarekHipError):
        hip.generate_source(MATCH_WITH_A_VARIABLE_PATTERN.replace("(? other)", "(? other more)"))


def test_the_program_model_on_the_references_known_answers(hip):
    """The integer cases of the reference's own unit tests for its IR walker (tests/interp_cases.py), through the
    tests' walker: the model the seeded programs are held to gives the reference's answers."""
    import numpy as np
    import interp_cases
    import ir_programs
    out = np.full(32, -7, np.int32)
    arrays = {"data": np.array([10, 20, 30], np.int32), "seven": np.zeros(7, np.int32), "out": out,
              "fout": np.zeros(1, np.float32)}
    ir_programs.evaluate(interp_cases.kernel(only_integers=True), arrays, 1)
    for k, want in interp_cases.EXPECTED.items():
        if k not in (3, 4, 7, 18):
            assert out[k] == want, k
    # and the whole kernel lowers to text the device compiler takes
    text = hip.generate_source(interp_cases.kernel())
    assert "int a[5] = {};" in text and "out[7] = (int)42.700000000000003f;" in text


def test_a_record_literal_that_reads_what_it_is_assigned_to(hip):
    """`ps.(i) <- {x = ps.(i).y; y = ps.(i).x}`: the reference stores field by field (Sarek_ir_cuda.ml:440-444), so
    the second field would read the first one's new value; OCaml builds the record first.  The values are taken
    before the first store when one of them names the target's vector or variable; otherwise the text is the
    reference's."""
    pt = "(record point (x i32) (y i32))"
    read = "(read ps (var i 2 i32))"
    swap = f"(assign (lelem ps (var i 2 i32)) (record point (x (field {read} y)) (y (field {read} x))))"
    params = f"(param (var ps 1 (vec {pt}))) (param (var i 2 i32)) (param (var qs 3 (vec {pt})))"
    ir = f"(kernel k (params {params}) (locals) (body {swap}) (types (point (x i32) (y i32))) (native_fn true))"
    text = hip.generate_source(ir)
    assert ("  {\n    const auto sarek_field_0 = ps[i].y;\n    const auto sarek_field_1 = ps[i].x;\n"
            "    ps[i].x = sarek_field_0;\n    ps[i].y = sarek_field_1;\n  }\n") in text
    other = ir.replace("(assign (lelem ps ", "(assign (lelem qs ")
    assert "  qs[i].x = ps[i].y;\n  qs[i].y = ps[i].x;\n" in hip.generate_source(other)
    # a variable whose name only contains the target's is not the target
    longer = other.replace("(var qs 3", "(var s 3").replace("(lelem qs ", "(lelem s ")
    assert "  s[i].x = ps[i].y;\n  s[i].y = ps[i].x;\n" in hip.generate_source(longer)
