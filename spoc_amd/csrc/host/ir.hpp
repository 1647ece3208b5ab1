// Kernel IR of the Sarek DSL as the plugin receives it, mirrored in C++.
// One node kind per constructor of the reference's ADT
// (spoc/ir/Sarek_ir_types.ml:12-245), so the lowering and the pattern matchers read
// like their OCaml counterparts.  The IR crosses the C ABI as an s-expression text
// (see ir_text.cpp for the grammar).
#pragma once
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace sarek_hip {
namespace ir {

enum class MemSpace { Global, Shared, Local };

struct Type;
using TypeP = std::shared_ptr<const Type>;
struct Type {
  enum Kind { Int32, Int64, Float32, Float64, Bool, Unit, Record, Variant, Array, Vec } kind = Unit;
  std::string name;                                                   // Record / Variant
  std::vector<std::pair<std::string, TypeP>> fields;                  // Record
  std::vector<std::pair<std::string, std::vector<TypeP>>> constrs;    // Variant
  TypeP elt;                                                          // Array / Vec
  MemSpace mem = MemSpace::Global;                                    // Array
};

struct Var {
  std::string name;
  int id = 0;
  TypeP type;
  bool is_mutable = false;
};

enum class Binop { Add, Sub, Mul, Div, Mod, Eq, Ne, Lt, Le, Gt, Ge, And, Or, Shl, Shr, BitAnd, BitOr, BitXor };
enum class Unop { Neg, Not, BitNot };

struct Pattern {
  bool wildcard = true;
  std::string constr;
  std::vector<std::string> vars;
};

struct Expr;
using ExprP = std::shared_ptr<const Expr>;
struct Expr {
  enum Kind {
    ConstInt32, ConstInt64, ConstFloat32, ConstFloat64, ConstBool, ConstUnit,
    VarRef, BinopE, UnopE, ArrayRead, ArrayReadExpr, RecordField, Intrinsic, Cast, Tuple, App,
    Record, Variant, ArrayLen, ArrayCreate, If, Match
  } kind = ConstUnit;
  int64_t ival = 0;            // ConstInt32 / ConstInt64 / ConstBool
  double fval = 0.0;           // ConstFloat32 / ConstFloat64
  Var var;                     // VarRef
  Binop binop = Binop::Add;
  Unop unop = Unop::Neg;
  std::string name;            // ArrayRead arr, RecordField field, Intrinsic name, Record/Variant type, ArrayLen arr
  std::string name2;           // Variant constructor
  std::vector<std::string> path;      // Intrinsic module path
  std::string templ;                  // Intrinsic: device template resolved by the caller's registry ("" = none)
  bool has_templ = false;
  std::vector<ExprP> args;            // operands / elements / call args, meaning depends on kind
  std::vector<std::pair<std::string, ExprP>> fields;   // Record construction
  TypeP type;                         // Cast target, ArrayCreate element type
  MemSpace mem = MemSpace::Global;    // ArrayCreate
  std::vector<std::pair<Pattern, ExprP>> cases;        // Match
};

struct LValue;
using LValueP = std::shared_ptr<const LValue>;
struct LValue {
  enum Kind { LVar, LArrayElem, LArrayElemExpr, LRecordField } kind = LVar;
  Var var;
  std::string name;   // array name / field name
  ExprP base, index;
  LValueP inner;      // LRecordField
};

struct Stmt;
using StmtP = std::shared_ptr<const Stmt>;
struct Stmt {
  enum Kind {
    Assign, Seq, If, While, For, Match, Return, Barrier, WarpBarrier, ExprS, Empty, Let, LetMut,
    Pragma, MemFence, Block, Native
  } kind = Empty;
  LValueP lhs;                 // Assign
  ExprP e, e2;                 // Assign rhs / cond / For lo,hi / Return / ExprS / Let init
  std::vector<StmtP> stmts;    // Seq; If: [then, else?]; While/For/Let/LetMut/Pragma/Block: [body]
  Var var;                     // For / Let / LetMut
  bool downto = false;         // For
  std::vector<std::pair<Pattern, StmtP>> cases;   // Match
  std::vector<std::string> hints;                 // Pragma
  std::string native_code;                        // Native: device text for this backend
};

struct Decl {
  enum Kind { Param, Local, Shared } kind = Param;
  Var var;                      // Param / Local
  bool has_array_info = false;  // Param
  TypeP arr_elt;
  MemSpace arr_mem = MemSpace::Global;
  ExprP init;                   // Local init / Shared size (may be null)
  std::string name;             // Shared
  TypeP elt;                    // Shared
};

struct HelperFunc {
  std::string name;
  std::vector<Var> params;
  TypeP ret;
  StmtP body;
};

struct Kernel {
  std::string name;
  std::vector<Decl> params, locals;
  StmtP body;
  std::vector<std::pair<std::string, std::vector<std::pair<std::string, TypeP>>>> types;
  std::vector<std::pair<std::string, std::vector<std::pair<std::string, std::vector<TypeP>>>>> variants;
  std::vector<HelperFunc> funcs;
  bool has_native_fn = false;   // kern_native_fn is Some _ (false for fused kernels)
};

// Errors of the text reader and of the lowering, carried to the C ABI as
// SAREK_HIP_E_PARSE / SAREK_HIP_E_CODEGEN.
struct ParseError : std::runtime_error {
  using std::runtime_error::runtime_error;
};
struct CodegenError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

// ir_text.cpp
Kernel parse_kernel(const std::string &text);
StmtP parse_stmt(const std::string &text);
ExprP parse_expr(const std::string &text);
std::string print_kernel(const Kernel &k);
std::string print_expr(const ExprP &e);
std::string print_stmt(const StmtP &s);

// ir_hip.cpp: IR -> HIP C++ for gfx950
std::string gen_expr(const ExprP &e);
std::string gen_stmt(const StmtP &s, const std::string &indent);
// For statements printed on their own (the body of a function some other text declares): the names that function
// already holds -- its parameters and locals -- so that a binding of one of them in the statements gets a name of
// its own, as inside generate().
struct FunctionScope {
  explicit FunctionScope(const std::vector<std::string> &names);
  ~FunctionScope();
  FunctionScope(const FunctionScope &) = delete;
  FunctionScope &operator=(const FunctionScope &) = delete;
};
// records + variants + helpers + kernel.  `block` (may be null): the launch block, when the
// caller knows it; sizes of shared arrays written in terms of the block dimensions
// (`let%shared tile = ()` lowers to block_dim_x elements, sarek/ppx/Sarek_lower_ir.ml:496-507)
// are then constants, which a __shared__ declaration needs.
std::string generate(const Kernel &k, const int block[3] = nullptr);

// specialise.cpp: "" or the tag of the hand-written kernel that computes the same thing
std::string recognise(const Kernel &k);
std::string canonical_form(const Kernel &k);   // the normal form recognise() compares

}  // namespace ir
}  // namespace sarek_hip
