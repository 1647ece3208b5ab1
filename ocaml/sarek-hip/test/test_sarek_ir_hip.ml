(* Unit tests of Sarek_ir_hip, the printer that turns Sarek IR into the s-expression text
   libsarek_hip.so lowers to HIP.  Where sarek-cuda/test/test_sarek_ir_cuda.ml:27-251 checks the
   CUDA text its generator prints for each statement form, the HIP plugin's OCaml side prints IR,
   not source, so each case here pins one constructor's form exactly: the reader on the other
   side (spoc_amd/csrc/host/ir_text.cpp) is strict, and a form that drifts is a launch that fails.
   The Python suite feeds every expected string of this file to that reader
   (tests/test_ocaml_veneer.py), which is what ties the two sides together without a compiler. *)
open Sarek_ir_types
module P = Sarek_hip.Sarek_ir_hip

let v ?(id = 0) ?(mut = false) name t = {var_name = name; var_id = id; var_type = t; var_mutable = mut}
let i n = EConst (CInt32 (Int32.of_int n))
let x = v ~id:1 "x" TInt32
let acc = v ~id:2 ~mut:true "acc" TFloat32

let table printer cases () =
  List.iter (fun (what, value, expected) -> Alcotest.(check string) what expected (printer value)) cases

let types =
  [ ("scalars", TVec TFloat32, "(vec f32)");
    ("int64 vector", TVec TInt64, "(vec i64)");
    ("shared array", TArray (TFloat64, Shared), "(array f64 shared)");
    ("record", TRecord ("point", [("x", TFloat32); ("y", TFloat32)]), "(record point (x f32) (y f32))");
    ("variant", TVariant ("shape", [("Circle", [TFloat32]); ("Empty", [])]), "(variant shape (Circle f32) (Empty))");
    ("bool and unit", TArray (TBool, Local), "(array bool local)") ]

let constants_and_variables =
  [ ("int32", EConst (CInt32 42l), "(i32 42)");
    ("negative int64", EConst (CInt64 (-7L)), "(i64 -7)");
    ("bool", EConst (CBool true), "(bool true)");
    ("unit", EConst CUnit, "(unit)");
    ("float32 keeps every digit", EConst (CFloat32 0.1), "(f32 0.10000000000000001)");
    ("immutable variable", EVar x, "(var x 1 i32)");
    ("mutable variable", EVar acc, "(var acc 2 f32 mut)") ]

let expressions =
  [ ("addition", EBinop (Add, i 1, i 2), "(add (i32 1) (i32 2))");
    ("comparison of a variable", EBinop (Lt, EVar x, i 10), "(lt (var x 1 i32) (i32 10))");
    ("shift and mask", EBinop (BitAnd, EBinop (Shr, EVar x, i 8), i 255), "(bitand (shr (var x 1 i32) (i32 8)) (i32 255))");
    ("negation", EUnop (Neg, EVar x), "(neg (var x 1 i32))");
    ("vector read", EArrayRead ("a", EVar x), "(read a (var x 1 i32))");
    ("field", ERecordField (EArrayRead ("ps", EVar x), "y"), "(field (read ps (var x 1 i32)) y)");
    ("cast", ECast (TFloat32, EVar x), "(cast f32 (var x 1 i32))");
    ("if expression", EIf (EConst (CBool true), i 1, i 2), "(if (bool true) (i32 1) (i32 2))");
    ("record literal", ERecord ("point", [("x", EConst (CFloat32 1.)); ("y", EConst (CFloat32 2.))]),
     "(record point (x (f32 1)) (y (f32 2)))");
    ("constructor with a payload", EVariant ("shape", "Circle", [EConst (CFloat32 2.)]), "(variant shape Circle (f32 2))");
    ("constructor without one", EVariant ("shape", "Empty", []), "(variant shape Empty)");
    ("vector length", EArrayLen "a", "(len a)");
    ("shared array of 256", EArrayCreate (TFloat32, i 256, Shared), "(newarray f32 (i32 256) shared)");
    ("match expression",
     EMatch (EVar (v ~id:3 "s" (TVariant ("shape", []))), [(PConstr ("Circle", ["r"]), i 1); (PWild, i 0)]),
     "(match (var s 3 (variant shape)) (case (Circle r) (i32 1)) (case _ (i32 0)))");
    ("match with a variable pattern",
     EMatch (EVar (v ~id:3 "s" (TVariant ("shape", []))), [(PConstr ("Circle", ["r"]), i 1); (PConstr ("", ["rest"]), i 0)]),
     "(match (var s 3 (variant shape)) (case (Circle r) (i32 1)) (case (? rest) (i32 0)))");
    ("helper call", EApp (EVar (v "square" TFloat32), [EVar acc]), "(app (var square 0 f32) (var acc 2 f32 mut))") ]

let statements =
  [ ("empty", SEmpty, "(empty)");
    ("sequence", SSeq [SEmpty; SBarrier], "(seq (empty) (barrier))");
    ("the three fences", SSeq [SBarrier; SWarpBarrier; SMemFence], "(seq (barrier) (warpbarrier) (memfence))");
    ("store to a vector", SAssign (LArrayElem ("a", EVar x), i 0), "(assign (lelem a (var x 1 i32)) (i32 0))");
    ("assignment to a mutable", SAssign (LVar acc, EConst (CFloat32 0.)), "(assign (lvar (var acc 2 f32 mut)) (f32 0))");
    ("field of an element", SAssign (LRecordField (LArrayElem ("ps", EVar x), "y"), EConst (CFloat32 1.)),
     "(assign (lfield (lelem ps (var x 1 i32)) y) (f32 1))");
    ("if without else", SIf (EConst (CBool true), SEmpty, None), "(if (bool true) (empty))");
    ("if with else", SIf (EConst (CBool false), SEmpty, Some SBarrier), "(if (bool false) (empty) (barrier))");
    ("while", SWhile (EBinop (Lt, EVar x, i 10), SEmpty), "(while (lt (var x 1 i32) (i32 10)) (empty))");
    ("for upto (inclusive bound)", SFor (x, i 0, i 9, Upto, SEmpty), "(for (var x 1 i32) (i32 0) (i32 9) upto (empty))");
    ("for downto", SFor (x, i 9, i 0, Downto, SEmpty), "(for (var x 1 i32) (i32 9) (i32 0) downto (empty))");
    ("return", SReturn (i 0), "(return (i32 0))");
    ("let", SLet (x, i 42, SEmpty), "(let (var x 1 i32) (i32 42) (empty))");
    ("mutable let", SLetMut (acc, EConst (CFloat32 0.), SEmpty), "(letmut (var acc 2 f32 mut) (f32 0) (empty))");
    ("block", SBlock SEmpty, "(block (empty))");
    ("pragma", SPragma (["unroll"], SEmpty), "(pragma (\"unroll\") (empty))");
    ("statement match", SMatch (EVar x, [(PWild, SEmpty)]), "(match (var x 1 i32) (case _ (empty)))");
    ("expression statement", SExpr (EVar x), "(expr (var x 1 i32))") ]

let test_kernel () =
  let a = v ~id:1 "a" (TVec TFloat32) and n = v ~id:2 "n" TInt32 in
  let k =
    { kern_name = "sarek_kern";
      kern_params = [DParam (a, Some {arr_elttype = TFloat32; arr_memspace = Global}); DParam (n, None)];
      kern_locals = []; kern_body = SEmpty; kern_types = [("point", [("x", TFloat32)])];
      kern_variants = [("shape", [("Empty", [])])]; kern_funcs = []; kern_native_fn = None } in
  Alcotest.(check string) "a whole kernel"
    "(kernel sarek_kern (params (param (var a 1 (vec f32)) (arr f32 global)) (param (var n 2 i32))) (locals) \
     (body (empty)) (types (point (x f32))) (variants (shape (Empty))) (funcs) (native_fn false))"
    (P.kernel k)

let test_intrinsic_without_a_template () =
  (* a name the registry does not hold travels bare; the native lowering knows the thread, barrier,
     atomic and math names itself *)
  Alcotest.(check string) "thread index" "(intr (Gpu) no_such_intrinsic_for_this_test)"
    (P.expr (EIntrinsic (["Gpu"], "no_such_intrinsic_for_this_test", [])))

let () =
  Alcotest.run "Sarek_ir_hip"
    [ ("types", [Alcotest.test_case "forms" `Quick (table P.ty types)]);
      ("expressions",
       [ Alcotest.test_case "constants and variables" `Quick (table P.expr constants_and_variables);
         Alcotest.test_case "operators, reads, literals" `Quick (table P.expr expressions);
         Alcotest.test_case "intrinsic without a registry template" `Quick test_intrinsic_without_a_template ]);
      ("statements", [Alcotest.test_case "forms" `Quick (table P.stmt statements)]);
      ("kernel", [Alcotest.test_case "whole kernel" `Quick test_kernel]) ]
