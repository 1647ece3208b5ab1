"""The IR fusion pass against the reference's own tests: every case of
sarek/tests/unit/test_fusion.ml (23) and sarek/tests/e2e/test_fusion_api.ml (3), with the same
kernels and the same assertions, plus exact-text checks of the rewrites worked out by hand from
sarek/sarek/Sarek_fusion.ml (each aimed at one plausible slip: wrong list order, wrong shift
sign, a parameter kept or dropped, a construct traversed that the reference leaves alone)."""
import pytest

from spoc_amd import fusion as F

TID = "(intr (Gpu) thread_idx_x)"          # test_fusion.ml:18


def mk_var(name, vid, ty="i32"):           # test_fusion.ml:13-15 (var_mutable = true)
    return f"(var {name} {vid} {ty} mut)"


def i32(n): return f"(i32 {n})"
def op(o, a, b): return f"({o} {a} {b})"
def read(arr, idx): return f"(read {arr} {idx})"
def store(arr, idx, e): return f"(assign (lelem {arr} {idx}) {e})"
def seq(*s): return "(seq " + " ".join(s) + ")"


def kernel(name, body, params=""):
    return f"(kernel {name} (params{params}) (locals) (body {body}) (native_fn false))"


def norm(text):
    return " ".join(text.split())


SCALE = store("temp", TID, op("mul", read("input", TID), i32(2)))          # temp[i] = input[i] * 2
PLUS1 = store("output", TID, op("add", read("temp", TID), i32(1)))         # output[i] = temp[i] + 1
PRODUCER, CONSUMER = kernel("producer", SCALE), kernel("consumer", PLUS1)
BARRIER_PRODUCER = kernel("producer", seq(store("temp", TID, read("input", TID)), "(barrier)"))
COPY_CONSUMER = kernel("consumer", store("output", TID, read("temp", TID)))
I, SUM = mk_var("i", 1), mk_var("sum", 2)
REDUCE_LOOP = f"(for {I} {i32(0)} {i32(100)} upto (assign (lvar {SUM}) (add {SUM} {read('temp', I)})))"
REDUCE = kernel("reduce", seq(f"(assign (lvar {SUM}) {i32(0)})", REDUCE_LOOP))
MAP = kernel("map", SCALE)
TEMP_3PT = op("add", op("add", read("temp", op("sub", TID, i32(1))), read("temp", TID)),
              read("temp", op("add", TID, i32(1))))
TEMP_2PT = op("add", read("temp", op("sub", TID, i32(1))), read("temp", op("add", TID, i32(1))))
K1 = kernel("k1", store("a", TID, op("mul", read("input", TID), i32(2))))
K2 = kernel("k2", store("b", TID, op("add", read("a", TID), i32(1))))
K3 = kernel("k3", store("output", TID, op("mul", read("b", TID), i32(3))))


# ---- sarek/tests/unit/test_fusion.ml, in its order -------------------------------------------

def test_expr_equal():                      # :266-274
    e1 = op("add", i32(1), i32(2))
    assert F.expr_equal(e1, op("add", i32(1), i32(2)))
    assert not F.expr_equal(e1, op("add", i32(1), i32(3)))
    assert F.expr_equal(TID, TID)


def test_subst_array_read():                # :277-293
    original = op("add", read("temp", TID), i32(1))
    replacement = op("mul", read("input", TID), i32(2))
    assert F.subst_array_read("temp", TID, replacement, original) == op("add", replacement, i32(1))


def test_analyze_one_to_one():              # :21-46
    info = F.analyze(kernel("scale", store("output", TID, op("mul", read("input", TID), i32(2)))))
    assert len(info.reads) == 1 and len(info.writes) == 1
    assert dict(info.reads)["input"] == ("OneToOne", TID)
    assert dict(info.writes)["output"] == ("OneToOne", TID)
    assert not info.has_barriers and not info.has_atomics


def test_analyze_with_barrier():            # :49-77
    body = seq(store("shared", TID, read("input", TID)), "(barrier)", store("output", TID, read("shared", TID)))
    assert F.analyze(kernel("with_barrier", body)).has_barriers


def test_can_fuse_compatible():             # :80-117
    assert F.can_fuse(PRODUCER, CONSUMER, "temp")


def test_can_fuse_with_barrier():           # :120-158
    assert not F.can_fuse(BARRIER_PRODUCER, COPY_CONSUMER, "temp")


def test_fuse_simple():                     # :161-207
    fused = F.fuse(PRODUCER, CONSUMER, "temp")
    assert fused.startswith("(kernel consumer_fused")
    info = F.analyze(fused)
    assert "temp" not in dict(info.reads) and "input" in dict(info.reads) and "output" in dict(info.writes)
    assert norm(store("output", TID, op("add", op("mul", read("input", TID), i32(2)), i32(1)))) in norm(fused)


def test_fuse_pipeline():                   # :210-263
    fused, eliminated = F.fuse_pipeline([K1, K2, K3])
    assert eliminated == ["b", "a"]          # consed: latest first
    info = F.analyze(fused)
    assert "input" in dict(info.reads) and "output" in dict(info.writes)
    assert "a" not in dict(info.reads) and "b" not in dict(info.reads)
    assert fused.startswith("(kernel k3_fused")
    expected = op("mul", op("add", op("mul", read("input", TID), i32(2)), i32(1)), i32(3))
    assert norm(store("output", TID, expected)) in norm(fused)


def test_detect_reduction_pattern():        # :296-317
    r = F.detect_reduction_pattern(
        f"(for {I} {i32(0)} {i32(100)} upto (assign (lvar {SUM}) (add {SUM} {read('arr', I)})))")
    assert r is not None and r.acc == "sum" and r.op == "add" and r.array == "arr" and r.loop_var == "i"


def test_is_reduction_kernel():             # :320-350
    assert F.is_reduction_kernel(kernel("reduce_sum", seq(f"(assign (lvar {SUM}) {i32(0)})", REDUCE_LOOP)),
                                 "temp") == "add"


def test_can_fuse_reduction():              # :353-394
    assert F.can_fuse_reduction(MAP, REDUCE, "temp")


def test_fuse_reduction():                  # :397-443
    fused = F.fuse_reduction(MAP, REDUCE, "temp")
    assert fused.startswith("(kernel reduce_fused")
    assert "temp" not in dict(F.analyze(fused).reads)


def test_try_fuse_reduction():              # :446-484
    assert F.try_fuse(MAP, REDUCE, "temp") is not None


def test_stencil_pattern():                 # :487-518
    blur = op("div", op("add", op("add", read("input", op("sub", TID, i32(1))), read("input", TID)),
                        read("input", op("add", TID, i32(1)))), i32(3))
    assert dict(F.analyze(kernel("blur", store("output", TID, blur))).reads)["input"] == ("Stencil", [-1, 0, 1])


def test_stencil_radius():                  # :521-526
    assert F.stencil_radius([-1, 0, 1]) == 1
    assert F.stencil_radius([-2, -1, 0, 1, 2]) == 2
    assert F.stencil_radius([0]) == 0
    assert F.stencil_radius([-3, 0, 1]) == 3


STENCIL_PRODUCER = kernel("producer", store("temp", TID, op("add", read("input", op("sub", TID, i32(1))),
                                                            read("input", op("add", TID, i32(1))))))


def test_can_fuse_stencil():                # :529-567
    assert F.can_fuse_stencil(STENCIL_PRODUCER, kernel("consumer", store("output", TID, TEMP_3PT)), "temp")


def test_fuse_stencil():                    # :570-606
    fused = F.fuse_stencil(PRODUCER, kernel("consumer", store("output", TID, TEMP_2PT)), "temp")
    assert fused.startswith("(kernel consumer_stencil_fused")
    assert "temp" not in dict(F.analyze(fused).reads)
    expected = op("add", op("mul", read("input", op("sub", TID, i32(1))), i32(2)),
                  op("mul", read("input", op("add", TID, i32(1))), i32(2)))
    assert norm(store("output", TID, expected)) in norm(fused)


def test_try_fuse_all():                    # :609-635
    assert F.try_fuse_all(PRODUCER, CONSUMER, "temp") is not None


def test_should_fuse_one_to_one():          # :638-664
    assert F.should_fuse(PRODUCER, CONSUMER, "temp") == (F.Fuse, "Element-wise producer/consumer")


def test_should_fuse_barrier():             # :667-695
    assert F.should_fuse(BARRIER_PRODUCER, COPY_CONSUMER, "temp") == (F.DontFuse, "Barrier prevents fusion")


def test_should_fuse_small_stencil():       # :698-730
    hint = F.should_fuse(PRODUCER, kernel("consumer", store("output", TID, TEMP_3PT)), "temp")
    assert hint == (F.MaybeFuse, "Small stencil - profile to decide")


def test_auto_fuse_pipeline():              # :733-776
    fused, eliminated, skipped = F.auto_fuse_pipeline([K1, K2, K3])
    assert "a" in eliminated and "b" in eliminated and skipped == []
    info = F.analyze(fused)
    assert "input" in dict(info.reads) and "output" in dict(info.writes)


def test_auto_fuse_pipeline_skip_stencil():  # :779-812
    k1 = kernel("k1", SCALE)
    k2 = kernel("k2", store("output", TID, TEMP_2PT))
    fused, eliminated, skipped = F.auto_fuse_pipeline([k1, k2])
    assert eliminated == [] and skipped == ["Small stencil - profile to decide"]
    assert fused.startswith("(kernel k2")      # the unfused consumer carries on


# ---- sarek/tests/e2e/test_fusion_api.ml: kernels as the PPX writes them (with parameters) ------

def ppx_kernel(name, out, inp, rhs):
    params = f" (param (var {out} 1 (vec i32))) (param (var {inp} 2 (vec i32)))"
    return kernel(name, store(out, TID, rhs), params)


API_PRODUCER = ppx_kernel("producer", "temp", "input", op("mul", read("input", TID), i32(2)))     # :11-14
API_CONSUMER = ppx_kernel("consumer", "output", "temp", op("add", read("temp", TID), i32(1)))     # :17-20


def test_api_can_fuse():                    # :29-39
    assert F.can_fuse(API_PRODUCER, API_CONSUMER, "temp")


def test_api_fuse():                        # :42-51
    fused = F.fuse(API_PRODUCER, API_CONSUMER, "temp")
    assert fused.startswith("(kernel consumer_fused")
    # consumer's parameters without the intermediate, then the producer's new ones (:490-540)
    assert norm("(params (param (var output 1 (vec i32))) (param (var input 2 (vec i32))))") in norm(fused)
    assert "(native_fn false)" in fused


def test_api_fuse_pipeline():               # :54-80
    s1 = ppx_kernel("stage1", "a", "input", op("mul", read("input", TID), i32(2)))
    s2 = ppx_kernel("stage2", "b", "a", op("add", read("a", TID), i32(1)))
    s3 = ppx_kernel("stage3", "output", "b", op("mul", read("b", TID), i32(3)))
    fused, eliminated = F.fuse_pipeline([s1, s2, s3])
    assert "a" in eliminated and "b" in eliminated
    assert fused.startswith("(kernel stage3_fused_fused") or fused.startswith("(kernel stage3_fused")
    assert norm("(params (param (var output 1 (vec i32))) (param (var input 2 (vec i32))))") in norm(fused)


# ---- what the source fixes beyond its tests ----------------------------------------------------

def test_pipeline_names_accumulate():
    # fuse k1 into k2 -> "k2_fused"; that into k3 -> "k3_fused" (consumer's name + suffix, :539)
    fused, _ = F.fuse_pipeline([K1, K2, K3])
    assert fused.startswith("(kernel k3_fused\n")
    two, _ = F.fuse_pipeline([K1, K2])
    assert two.startswith("(kernel k2_fused\n")


def test_expr_equal_looks_at_few_forms_only():
    # :35-48: variables by id (names ignored); casts, fields, tuples ... never compare equal
    assert F.expr_equal("(var x 3 i32)", "(var y 3 i32)")
    assert not F.expr_equal("(var x 3 i32)", "(var x 4 i32)")
    cast = f"(cast i64 {TID})"
    assert not F.expr_equal(cast, cast)
    assert not F.expr_equal("(tuple (i32 1))", "(tuple (i32 1))")
    assert not F.expr_equal(i32(1), "(i64 1)")
    assert F.expr_equal("(f32 0.0)", "(f32 -0.0)") and not F.expr_equal("(f32 nan)", "(f32 nan)")
    assert F.expr_equal("(neg (intr (Gpu) f x))".replace(" x", f" {i32(1)}"), f"(neg (intr (Gpu) f {i32(1)}))")
    assert not F.expr_equal(f"(intr (Gpu) f {i32(1)})", f"(intr (Std) f {i32(1)})")


def test_subst_leaves_array_creation_alone_and_enters_indices():
    # :80-81 index of another read is rewritten; :108 the size of an array creation is not
    e = read("other", read("temp", TID))
    assert F.subst_array_read("temp", TID, i32(7), e) == read("other", i32(7))
    create = f"(newarray i32 {read('temp', TID)} shared)"
    assert F.subst_array_read("temp", TID, i32(7), create) == create
    # a read of the array at another index stays
    other_idx = read("temp", op("add", TID, i32(1)))
    assert F.subst_array_read("temp", TID, i32(7), other_idx) == other_idx


def test_conditional_producer_store_is_not_inlined():
    # find_write_expr gives up on conditionals (:370-372): fuse returns the consumer itself
    guarded = kernel("producer", f"(if (lt {TID} (i32 10)) {SCALE})")
    assert F.can_fuse(guarded, CONSUMER, "temp")           # the analysis still says yes
    fused = F.fuse(guarded, CONSUMER, "temp")
    assert fused.startswith("(kernel consumer\n") and norm(PLUS1) in norm(fused)


def test_first_store_in_a_sequence_wins():
    # :363-369
    two = kernel("producer", seq(store("temp", TID, i32(1)), store("temp", TID, i32(2))))
    fused = F.fuse(two, CONSUMER, "temp")
    assert norm(store("output", TID, op("add", i32(1), i32(1)))) in norm(fused)


def test_index_of_the_consumer_read_found_first_in_list_order():
    # collect_reads conses: the LAST read in evaluation order heads the list (:198-266), and
    # fuse takes the head (:463-467).  Consumer reads temp[i+1] then temp[i]: idx = i.
    cons = kernel("consumer", store("output", TID, op("add", read("temp", op("add", TID, i32(1))),
                                                      read("temp", TID))))
    fused = F.fuse(PRODUCER, cons, "temp")
    expected = op("add", read("temp", op("add", TID, i32(1))), op("mul", read("input", TID), i32(2)))
    assert norm(store("output", TID, expected)) in norm(fused)
    # the other way round the head is temp[i+1], which the producer never stores: unchanged
    cons2 = kernel("consumer", store("output", TID, op("add", read("temp", TID),
                                                       read("temp", op("add", TID, i32(1))))))
    assert F.fuse(PRODUCER, cons2, "temp").startswith("(kernel consumer\n")


def test_reduction_rewrite_inserts_the_producer_expression_as_it_stands():
    # :693-699: arr[loop_var] -> the producer's right-hand side, still indexed by thread_idx_x
    fused = F.fuse_reduction(MAP, REDUCE, "temp")
    expected = f"(assign (lvar {SUM}) (add {SUM} {op('mul', read('input', TID), i32(2))}))"
    assert norm(expected) in norm(fused)
    # operands the other way round are recognised too (:619-621), downto loops are not (:614)
    flipped = REDUCE_LOOP.replace(f"(add {SUM} {read('temp', I)})", f"(add {read('temp', I)} {SUM})")
    assert F.detect_reduction_pattern(flipped).array == "temp"
    assert F.detect_reduction_pattern(REDUCE_LOOP.replace("upto", "downto")) is None
    # a loop inside a let is not looked at by is_reduction_kernel (:627-634)
    hidden = kernel("reduce", f"(letmut {SUM} {i32(0)} {REDUCE_LOOP})")
    assert F.is_reduction_kernel(hidden, "temp") is None
    assert not F.can_fuse_reduction(MAP, hidden, "temp")


def test_stencil_of_stencil_shifts_compose():
    # :876-926: temp[i-1] -> producer expression shifted by -1: input[(i-1)-1] + input[(i+1)-1]
    cons = kernel("consumer", store("output", TID, TEMP_3PT))
    fused = F.fuse_stencil(STENCIL_PRODUCER, cons, "temp")

    def shifted(k):
        lo, hi = op("sub", TID, i32(1)), op("add", TID, i32(1))
        if k == 0:
            return op("add", read("input", lo), read("input", hi))
        w = (lambda e: op("add", e, i32(k))) if k > 0 else (lambda e: op("sub", e, i32(-k)))
        return op("add", read("input", w(lo)), read("input", w(hi)))
    expected = op("add", op("add", shifted(-1), shifted(0)), shifted(1))
    assert norm(store("output", TID, expected)) in norm(fused)
    info = F.analyze_stencil_fusion(STENCIL_PRODUCER, cons, "temp")
    assert info == (2, 1, 1, ["input"])
    assert F.analyze_stencil_fusion(PRODUCER, CONSUMER, "temp") == (0, 0, 0, ["input"])


def test_stencil_offset_forms():
    # extract_offset (:284-289): base+c, base-c, c+base; c-base is not an offset -> Gather
    def reads(*idx):
        body = i32(0)
        for i in idx:
            body = op("add", body, read("in", i))
        return dict(F.analyze(kernel("k", store("out", TID, body))).reads)["in"]
    assert reads(op("add", TID, i32(2)), op("add", i32(3), TID), op("sub", TID, i32(1)), TID) == \
        ("Stencil", [-1, 0, 2, 3])
    assert reads(op("sub", i32(1), TID), TID) == ("Gather", None)
    assert reads(op("add", "(var j 9 i32)", i32(1)), TID) == ("Gather", None)       # different bases
    assert reads(op("add", TID, i32(1)), op("add", TID, i32(1))) == ("Stencil", [1])   # duplicates collapse


def test_two_reads_of_one_element_are_a_stencil():
    # :296-322: more than one read -> never OneToOne, so can_fuse says no and the stencil path takes it
    square = kernel("square", store("output", TID, op("mul", read("temp", TID), read("temp", TID))))
    assert dict(F.analyze(square).reads)["temp"] == ("Stencil", [0])
    assert not F.can_fuse(PRODUCER, square, "temp") and F.try_fuse(PRODUCER, square, "temp") is None
    assert F.should_fuse(PRODUCER, square, "temp").decision == F.MaybeFuse
    fused = F.try_fuse_all(PRODUCER, square, "temp")
    scaled = op("mul", read("input", TID), i32(2))
    assert fused.startswith("(kernel square_stencil_fused") and norm(op("mul", scaled, scaled)) in norm(fused)


def test_should_fuse_other_rules():         # :1087-1098
    five = TEMP_3PT
    for k in (2, 3):
        five = op("add", five, read("temp", op("add", TID, i32(k))))
    assert F.should_fuse(PRODUCER, kernel("c", store("output", TID, five)), "temp") == \
        (F.DontFuse, "Large stencil radius - keep separate")
    gather = op("add", read("temp", read("idx", TID)), read("temp", TID))
    assert F.should_fuse(PRODUCER, kernel("c", store("output", TID, gather)), "temp") == \
        (F.DontFuse, "Gather pattern - keep separate")
    assert F.should_fuse(PRODUCER, kernel("c", store("output", TID, read("input", TID))), "temp") == \
        (F.MaybeFuse, "Unknown pattern - profile to decide")


def test_analyze_pipeline_text():           # :1180-1214
    text = F.analyze_pipeline([K1, K2, kernel("k3", store("output", TID, TEMP_2PT.replace("temp", "b")))])
    assert text == ("=== Fusion Analysis ===\n"
                    "\n[0] k1 -> k2\n  [FUSE] via 'a': Element-wise producer/consumer\n"
                    "\n[1] k2 -> k3\n  [MAYBE] via 'b': Small stencil - profile to decide\n"
                    "\n")
    assert F.analyze_pipeline([K1]) == "=== Fusion Analysis ===\n\n"


def test_empty_pipeline_is_an_error():      # :573-574, :1137-1138; Fusion_error.ml:35-36
    with pytest.raises(F.FusionError, match="fuse_pipeline: cannot fuse empty kernel list"):
        F.fuse_pipeline([])
    with pytest.raises(F.FusionError, match="auto_fuse_pipeline: cannot fuse empty kernel list"):
        F.auto_fuse_pipeline([])
    only, eliminated = F.fuse_pipeline([K1])
    assert eliminated == [] and only.startswith("(kernel k1\n")


def test_merged_kernel_carries_locals_types_and_helpers():
    # :538-547: consumer's first, then the producer's; shared declarations are parameters too
    prod = ("(kernel p (params (param (var temp 1 (vec f32))) (param (var input 2 (vec f32))) "
            "(shared tile f32 (i32 64)) (param (var n 3 i32)))"
            " (locals (local (var pl 10 i32)))"
            f" (body {store('temp', TID, read('input', TID))})"
            " (types (ptype (x f32))) (funcs (func pf (params (var q 11 f32)) f32 (return (var q 11 f32))))"
            " (native_fn true))")
    cons = ("(kernel c (params (param (var out 4 (vec f32))) (param (var temp 1 (vec f32))) (param (var n 3 i32)))"
            " (locals (local (var cl 12 i32)))"
            f" (body {store('out', TID, read('temp', TID))})"
            " (types (ctype (y i32))) (native_fn true))")
    fused = norm(F.fuse(prod, cons, "temp"))
    assert ("(params (param (var out 4 (vec f32))) (param (var n 3 i32)) (param (var input 2 (vec f32))) "
            "(shared tile f32 (i32 64)))") in fused
    assert "(locals (local (var cl 12 i32)) (local (var pl 10 i32)))" in fused
    assert "(types (ctype (y i32)) (ptype (x f32)))" in fused
    assert "(func pf" in fused and "(native_fn false)" in fused


def test_bad_ir_is_a_parse_error():
    from spoc_amd import hip
    with pytest.raises(hip.SarekHipError) as e:
        F.analyze("(kernel k (params) (locals) (body (frobnicate)))")
    assert e.value.status == hip.E_PARSE
