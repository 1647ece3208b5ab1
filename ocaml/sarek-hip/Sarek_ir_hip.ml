(* Sarek IR -> the s-expression text libsarek_hip.so lowers to HIP (sarek_hip_generate_source).
   The lowering itself and the recogniser of the hot kernels are native; this module only prints
   the IR: one function per type of spoc/ir/Sarek_ir_types.ml, one form per constructor.  The
   reader on the other side is spoc_amd/csrc/host/ir_text.cpp, whose header holds the grammar.
   (The CUDA plugin generates source in OCaml instead, sarek-cuda/Sarek_ir_cuda.ml.)

   The S conversion of Printf escapes the double quote and the backslash the way the reader undoes
   them (it also knows the n and t escapes); OCaml's decimal escapes for other control characters do
   not occur in kernel text.  The reader bounds nesting at 2000 levels (each let adds one). *)
open Sarek_ir_types
let cat f l = String.concat "" (List.map (fun x -> " " ^ f x) l)       (* " a b c" *)
let mem = function Global -> "global" | Shared -> "shared" | Local -> "local"
let rec ty = function
  | TInt32 -> "i32" | TInt64 -> "i64" | TFloat32 -> "f32" | TFloat64 -> "f64" | TBool -> "bool" | TUnit -> "unit"
  | TVec t -> Printf.sprintf "(vec %s)" (ty t)
  | TArray (t, m) -> Printf.sprintf "(array %s %s)" (ty t) (mem m)
  | TRecord (n, fs) -> Printf.sprintf "(record %s%s)" n (cat (fun (f, t) -> Printf.sprintf "(%s %s)" f (ty t)) fs)
  | TVariant (n, cs) -> Printf.sprintf "(variant %s%s)" n (cat (fun (c, ts) -> Printf.sprintf "(%s%s)" c (cat ty ts)) cs)
let var v = Printf.sprintf "(var %s %d %s%s)" v.var_name v.var_id (ty v.var_type) (if v.var_mutable then " mut" else "")
let binop = function
  | Add -> "add" | Sub -> "sub" | Mul -> "mul" | Div -> "div" | Mod -> "mod" | Eq -> "eq" | Ne -> "ne" | Lt -> "lt"
  | Le -> "le" | Gt -> "gt" | Ge -> "ge" | And -> "and" | Or -> "or" | Shl -> "shl" | Shr -> "shr"
  | BitAnd -> "bitand" | BitOr -> "bitor" | BitXor -> "bitxor"
let unop = function Neg -> "neg" | Not -> "not" | BitNot -> "bitnot"
let pat = function
  | PWild -> "_"
  | PConstr ("", vs) -> Printf.sprintf "(?%s)" (cat Fun.id vs)   (* a variable pattern, Sarek_lower_ir.ml:559 *)
  | PConstr (c, vs) -> Printf.sprintf "(%s%s)" c (cat Fun.id vs)
let const = function
  | CInt32 n -> Printf.sprintf "(i32 %ld)" n | CInt64 n -> Printf.sprintf "(i64 %Ld)" n
  | CFloat32 f -> Printf.sprintf "(f32 %.17g)" f | CFloat64 f -> Printf.sprintf "(f64 %.17g)" f   (* nan, inf, -inf pass *)
  | CBool b -> Printf.sprintf "(bool %b)" b | CUnit -> "(unit)"
let rec expr = function
  | EConst c -> const c
  | EVar v -> var v
  | EBinop (op, a, b) -> Printf.sprintf "(%s %s %s)" (binop op) (expr a) (expr b)
  | EUnop (op, a) -> Printf.sprintf "(%s %s)" (unop op) (expr a)
  | EArrayRead (a, i) -> Printf.sprintf "(read %s %s)" a (expr i)
  | EArrayReadExpr (b, i) -> Printf.sprintf "(readx %s %s)" (expr b) (expr i)
  | ERecordField (e, f) -> Printf.sprintf "(field %s %s)" (expr e) f
  | EIntrinsic (path, name, args) ->
      (* what the registry holds for this intrinsic travels with it; thread / barrier / atomic / math names are
         intercepted natively first, as Sarek_ir_cuda.gen_intrinsic does (:238-348) *)
      let templ = match Sarek_registry.fun_device_template ~module_path:path name with
        | Some t -> Printf.sprintf " (template %S)" t | None -> "" in
      Printf.sprintf "(intr (%s) %s%s%s)" (String.concat " " path) name templ (cat expr args)
  | ECast (t, e) -> Printf.sprintf "(cast %s %s)" (ty t) (expr e)
  | ETuple es -> Printf.sprintf "(tuple%s)" (cat expr es)
  | EApp (f, args) -> Printf.sprintf "(app %s%s)" (expr f) (cat expr args)
  | ERecord (n, fs) -> Printf.sprintf "(record %s%s)" n (cat (fun (f, e) -> Printf.sprintf "(%s %s)" f (expr e)) fs)
  | EVariant (t, c, args) -> Printf.sprintf "(variant %s %s%s)" t c (cat expr args)
  | EArrayLen a -> Printf.sprintf "(len %s)" a
  | EArrayCreate (t, n, m) -> Printf.sprintf "(newarray %s %s %s)" (ty t) (expr n) (mem m)
  | EIf (c, a, b) -> Printf.sprintf "(if %s %s %s)" (expr c) (expr a) (expr b)
  | EMatch (e, cases) -> Printf.sprintf "(match %s%s)" (expr e) (cat (fun (p, e) -> Printf.sprintf "(case %s %s)" (pat p) (expr e)) cases)
let rec lvalue = function
  | LVar v -> Printf.sprintf "(lvar %s)" (var v)
  | LArrayElem (a, i) -> Printf.sprintf "(lelem %s %s)" a (expr i)
  | LArrayElemExpr (b, i) -> Printf.sprintf "(lelemx %s %s)" (expr b) (expr i)
  | LRecordField (l, f) -> Printf.sprintf "(lfield %s %s)" (lvalue l) f
let rec stmt = function
  | SAssign (lv, e) -> Printf.sprintf "(assign %s %s)" (lvalue lv) (expr e)
  | SSeq l -> Printf.sprintf "(seq%s)" (cat stmt l)
  | SIf (c, t, None) -> Printf.sprintf "(if %s %s)" (expr c) (stmt t)
  | SIf (c, t, Some e) -> Printf.sprintf "(if %s %s %s)" (expr c) (stmt t) (stmt e)
  | SWhile (c, s) -> Printf.sprintf "(while %s %s)" (expr c) (stmt s)
  | SFor (v, a, b, d, s) ->
      Printf.sprintf "(for %s %s %s %s %s)" (var v) (expr a) (expr b) (match d with Upto -> "upto" | Downto -> "downto") (stmt s)
  | SMatch (e, cases) -> Printf.sprintf "(match %s%s)" (expr e) (cat (fun (p, s) -> Printf.sprintf "(case %s %s)" (pat p) (stmt s)) cases)
  | SReturn e -> Printf.sprintf "(return %s)" (expr e)
  | SBarrier -> "(barrier)" | SWarpBarrier -> "(warpbarrier)" | SMemFence -> "(memfence)" | SEmpty -> "(empty)"
  | SExpr e -> Printf.sprintf "(expr %s)" (expr e)
  | SLet (v, e, s) -> Printf.sprintf "(let %s %s %s)" (var v) (expr e) (stmt s)
  | SLetMut (v, e, s) -> Printf.sprintf "(letmut %s %s %s)" (var v) (expr e) (stmt s)
  | SPragma (hints, s) -> Printf.sprintf "(pragma (%s) %s)" (String.concat " " (List.map (Printf.sprintf "%S") hints)) (stmt s)
  | SBlock s -> Printf.sprintf "(block %s)" (stmt s)
  | SNative {gpu; _} -> Printf.sprintf "(native %S)" (gpu ~framework:"HIP")
let decl = function
  | DParam (v, None) -> Printf.sprintf "(param %s)" (var v)
  | DParam (v, Some a) -> Printf.sprintf "(param %s (arr %s %s))" (var v) (ty a.arr_elttype) (mem a.arr_memspace)
  | DLocal (v, None) -> Printf.sprintf "(local %s)" (var v)
  | DLocal (v, Some e) -> Printf.sprintf "(local %s %s)" (var v) (expr e)
  | DShared (n, t, None) -> Printf.sprintf "(shared %s %s)" n (ty t)
  | DShared (n, t, Some e) -> Printf.sprintf "(shared %s %s %s)" n (ty t) (expr e)
let func f = Printf.sprintf "(func %s (params%s) %s %s)" f.hf_name (cat var f.hf_params) (ty f.hf_ret_type) (stmt f.hf_body)
let kernel k =
  Printf.sprintf "(kernel %s (params%s) (locals%s) (body %s) (types%s) (variants%s) (funcs%s) (native_fn %b))"
    k.kern_name (cat decl k.kern_params) (cat decl k.kern_locals) (stmt k.kern_body)
    (cat (fun (n, fs) -> Printf.sprintf "(%s%s)" n (cat (fun (f, t) -> Printf.sprintf "(%s %s)" f (ty t)) fs)) k.kern_types)
    (cat (fun (n, cs) -> Printf.sprintf "(%s%s)" n (cat (fun (c, ts) -> Printf.sprintf "(%s%s)" c (cat ty ts)) cs)) k.kern_variants)
    (cat func k.kern_funcs) (k.kern_native_fn <> None)
