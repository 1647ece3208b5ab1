"""The known answers of the reference's unit tests for its IR walker (sarek/tests/unit/test_ir_interp.ml:29-345), as
one kernel: thread 0 evaluates each case's expression or statements and stores the result.  `data` is the vector
[10, 20, 30], `seven` one of seven elements; `out` takes the int32 results, `fout` the float32 one.  EXPECTED maps
an index of `out` to what the reference's test asserts (a bool as 1 / 0, as its to_int32 gives them :332-337)."""

I = "(var i 20 i32 mut)"
SUM = "(var sum 21 i32 mut)"
X = "(var x 22 i32)"
POINT = "(record point (x i32) (y i32))"
OPTION = "(variant option (Some i32) (None))"


def out(k, e):
    return f"(assign (lelem out (i32 {k})) {e})"


CASES = [
    # (index in out, statement that stores it, the reference's expected value, test_ir_interp.ml lines)
    (0, out(0, "(read data (i32 1))"), 20, "29-52"),
    (1, out(1, "(len seven)"), 7, "88-99"),
    (2, f"(let (var a 23 (array i32 local)) (newarray i32 (i32 5) local) {out(2, '(read a (i32 0))')})", 0, "64-86"),
    (3, f"(let (var p 24 {POINT}) (record point (x (i32 10)) (y (i32 20))) {out(3, f'(field (var p 24 {POINT}) x)')})", 10, "101-126"),
    (4, f"(let (var v 25 {OPTION}) (variant option Some (i32 42)) (match (var v 25 {OPTION}) "
        f"(case (Some n) {out(4, '(var n 26 i32)')}) (case _ {out(4, '(i32 -1)')})))", 42, "128-150"),
    (5, out(5, "(if (bool true) (i32 10) (i32 20))"), 10, "155-164"),
    (6, out(6, "(if (bool false) (i32 10) (i32 20))"), 20, "166-175"),
    (7, out(7, "(cast i32 (f32 42.7))"), 42, "188-195"),
    (8, out(8, "(add (i32 10) (i32 20))"), 30, "199-206"),
    (9, out(9, "(mul (i32 5) (i32 7))"), 35, "208-215"),
    (10, out(10, "(cast i32 (lt (i32 10) (i32 20)))"), 1, "217-224"),
    (11, out(11, "(cast i32 (eq (i32 42) (i32 42)))"), 1, "226-233"),
    (12, out(12, "(neg (i32 42))"), -42, "237-244"),
    (13, out(13, "(cast i32 (not (bool true)))"), 0, "246-253"),
    (14, out(14, "(i32 99)"), 99, "257-269"),
    (15, f"(let {X} (i32 42) {out(15, X)})", 42, "271-282"),
    (16, f"(letmut {I} (i32 0) (seq (while (lt {I} (i32 3)) (assign (lvar {I}) (add {I} (i32 1)))) {out(16, I)}))", 3, "293-310"),
    (17, f"(letmut {SUM} (i32 0) (seq (for (var i 27 i32 mut) (i32 0) (i32 4) upto "
         f"(assign (lvar {SUM}) (add {SUM} (var i 27 i32 mut)))) {out(17, SUM)}))", 10, "312-328"),
    (18, out(18, "(cast i32 (f32 42.9))"), 42, "335"),
    (19, out(19, "(cast i32 (bool true))"), 1, "336"),
    (20, out(20, "(cast i32 (bool false))"), 0, "337"),
    (21, out(21, "(if (i32 42) (i32 1) (i32 0))"), 1, "343"),
    (22, out(22, "(if (i32 0) (i32 1) (i32 0))"), 0, "344"),
]
FLOAT_CASE = "(assign (lelem fout (i32 0)) (cast f32 (i32 42)))"      # 42.0, test_ir_interp.ml:179-186
EXPECTED = {k: want for k, _, want, _ in CASES}


def kernel(only_integers=False):
    """The kernel; with only_integers the record, variant and float cases are left out (the tests' own walker of the
    IR computes in integers)."""
    stmts = [s for k, s, _, _ in CASES if not (only_integers and k in (3, 4, 7, 18))]
    if not only_integers:
        stmts.append(FLOAT_CASE)
    return ("(kernel sarek_kern (params (param (var data 1 (vec i32))) (param (var seven 2 (vec i32))) "
            "(param (var out 3 (vec i32))) (param (var fout 4 (vec f32)))) (locals) "
            f"(body (if (eq (intr (Std) global_thread_id) (i32 0)) (seq {' '.join(stmts)}))) "
            "(types (point (x i32) (y i32))) (variants (option (Some i32) (None))) (native_fn true))")
