// IR -> HIP C++ lowering for gfx950 (the plugin's Sarek_ir_hip).
//
// Same surface rules as the reference's CUDA lowering so that kernels keep their
// meaning (sarek-cuda/Sarek_ir_cuda.ml): fully parenthesised binary and unary
// expressions (:96-106, :210-231), float32 literals as "%.17g" with a forced decimal
// point and an `f` suffix (:83-89), inclusive `for` loops (`<=` / `>=`, :474-496),
// vector parameters expanded to `T* __restrict__ v, int sarek_v_length` (:662-683),
// thread and barrier intrinsics resolved by name before any registry template
// (:232-267), records as typedef structs and variants as tag + union with make_*
// constructors (:796-868), everything inside one `extern "C" { }` block (:746-748).
//
// HIP-specific spellings: `__syncwarp()` does not exist for AMD targets, a wave-level
// barrier is `__builtin_amdgcn_wave_barrier()`; the source is compiled by hiprtc, which
// pre-includes the HIP device runtime, so no #include lines are emitted.
#include <algorithm>
#include <cctype>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <memory>
#include <utility>

#include "ir.hpp"

namespace sarek_hip {
namespace ir {
namespace {

// Variant definitions of the kernel being generated (for match bindings).
thread_local const Kernel *t_kernel = nullptr;
// Launch block known to the caller of generate (0 = unknown) and whether the expression being
// printed is the size of a shared array: there blockDim.* has to be a constant for the
// declaration to compile, so the known value is written instead.
thread_local int t_block[3] = {0, 0, 0};
thread_local bool t_in_shared_size = false;

// Names and C scopes.  The reference prints a let as `type name = value;` followed by its body in the same C block
// (sarek-cuda/Sarek_ir_cuda.ml:437-578), so a kernel that binds a name again -- `let x = f x in ...`, ordinary OCaml --
// comes out as a redefinition (or, in an inner block, as `int x = (x + 1);`, whose right-hand side is the new,
// uninitialised x) and does not compile there.  Here a binding whose name is already declared in an open C block of
// the function, or is one of its parameters, is printed under a name of its own (x_2, x_3, ...) for the length of its
// body; the value is printed first, with the outer meaning of the name.  A kernel without such a binding -- every
// golden text -- comes out as the reference prints it.
struct Rename {
  std::string name;
  int id;   // the binding's id in the IR, -1 where the IR gives none (a pattern's variables)
  std::string printed;
  bool is_mutable;   // a loop's own counter is not: only its loop changes it, between turns
};
thread_local std::vector<std::vector<std::string>> t_c_blocks;   // declared names per open C block
thread_local std::vector<Rename> t_renames;                      // innermost binding last

bool name_declared(const std::string &n) {
  for (const auto &block : t_c_blocks)
    for (const auto &d : block)
      if (d == n) return true;
  return false;
}

// What a use of the name prints: the binding of that name and id (the front end numbers every binding, so a use
// carries the id of the binding it means, sarek/ppx/Sarek_lower_ir.ml:237); where no binding in force has the id --
// an array use, which carries a name alone, or IR written by hand -- the innermost binding of the name.
const Rename *binding_of(const std::string &n, int id) {
  if (id >= 0)
    for (auto it = t_renames.rbegin(); it != t_renames.rend(); ++it)
      if (it->id == id && it->name == n) return &*it;
  for (auto it = t_renames.rbegin(); it != t_renames.rend(); ++it)
    if (it->name == n) return &*it;
  return nullptr;
}
const std::string &printed_name(const std::string &n, int id = -1) {
  const Rename *b = binding_of(n, id);
  return b ? b->printed : n;
}
const std::string &printed_name(const Var &v) { return printed_name(v.name, v.id); }

struct CBlock {   // an opening brace of the generated text
  size_t renames;
  CBlock() : renames(t_renames.size()) { t_c_blocks.emplace_back(); }
  ~CBlock() {
    t_c_blocks.pop_back();
    t_renames.erase(t_renames.begin() + static_cast<std::ptrdiff_t>(std::min(renames, t_renames.size())), t_renames.end());
  }
};

struct Binding {  // a declaration in the current C block; its name means the new variable while this object lives
  std::string printed;
  size_t at = 0;
  bool pushed = false;
  explicit Binding(const Var &v, bool is_mutable = false) : Binding(v.name, v.id, is_mutable || v.is_mutable) {}
  explicit Binding(const std::string &name, int id = -1, bool is_mutable = false) : printed(name) {
    if (t_c_blocks.empty()) return;   // a statement printed outside any function: nothing to compare with
    if (name_declared(name)) {
      int k = 2;
      do printed = name + "_" + std::to_string(k++);
      while (name_declared(printed));
    }
    t_c_blocks.back().push_back(printed);
    // the name stands for this variable in the body even when it is printed as it is: an outer rename of the same
    // name must not reach into it
    at = t_renames.size();
    t_renames.push_back({name, id, printed, is_mutable});
    pushed = true;
  }
  // A let without a body, in sequence with what uses it (a module's constant in front of the kernel function,
  // sarek/ppx/Sarek_lower_ir.ml:634-671): the name keeps this meaning until the C block closes.
  void keep() { pushed = false; }
  ~Binding() {
    if (pushed && at < t_renames.size()) t_renames.erase(t_renames.begin() + static_cast<std::ptrdiff_t>(at), t_renames.end());
  }
  Binding(const Binding &) = delete;
  Binding &operator=(const Binding &) = delete;
};

std::string mangle(const std::string &name) {
  std::string o = name;
  for (char &c : o)
    if (c == '.') c = '_';
  return o;
}

std::string type_str(const TypeP &t) {
  switch (t->kind) {
    case Type::Int32: return "int";
    case Type::Int64: return "long long";
    case Type::Float32: return "float";
    case Type::Float64: return "double";
    case Type::Bool: return "int";
    case Type::Unit: return "void";
    case Type::Record:
    case Type::Variant: return mangle(t->name);
    case Type::Array:
    case Type::Vec: return type_str(t->elt) + "*";
  }
  return "void";
}

std::string param_type_str(const TypeP &t) {
  if (t->kind == Type::Vec) return type_str(t->elt) + "* __restrict__";
  if (t->kind == Type::Array) return type_str(t->elt) + "*";
  return type_str(t);
}

const char *thread_intrinsic(const std::string &n) {
  if (t_in_shared_size && n.size() == 11 && n.compare(0, 10, "block_dim_") == 0) {
    const int axis = n[10] - 'x';
    if (axis >= 0 && axis < 3 && t_block[axis] > 0) {
      static thread_local char num[3][16];
      std::snprintf(num[axis], sizeof(num[axis]), "%d", t_block[axis]);
      return num[axis];
    }
  }
  static const struct {
    const char *name, *code;
  } table[] = {
      {"thread_id_x", "threadIdx.x"}, {"thread_idx_x", "threadIdx.x"},
      {"thread_id_y", "threadIdx.y"}, {"thread_idx_y", "threadIdx.y"},
      {"thread_id_z", "threadIdx.z"}, {"thread_idx_z", "threadIdx.z"},
      {"block_id_x", "blockIdx.x"}, {"block_idx_x", "blockIdx.x"},
      {"block_id_y", "blockIdx.y"}, {"block_idx_y", "blockIdx.y"},
      {"block_id_z", "blockIdx.z"}, {"block_idx_z", "blockIdx.z"},
      {"block_dim_x", "blockDim.x"}, {"block_dim_y", "blockDim.y"}, {"block_dim_z", "blockDim.z"},
      {"grid_dim_x", "gridDim.x"}, {"grid_dim_y", "gridDim.y"}, {"grid_dim_z", "gridDim.z"},
      {"global_thread_id", "(threadIdx.x + blockIdx.x * blockDim.x)"},
      {"global_idx", "(threadIdx.x + blockIdx.x * blockDim.x)"},
      {"global_idx_x", "(threadIdx.x + blockIdx.x * blockDim.x)"},
      {"global_idx_y", "(threadIdx.y + blockIdx.y * blockDim.y)"},
      {"global_idx_z", "(threadIdx.z + blockIdx.z * blockDim.z)"},
      {"global_size", "(blockDim.x * gridDim.x)"},
  };
  for (const auto &e : table)
    if (n == e.name) return e.code;
  return nullptr;
}

// Device templates of the standard-library intrinsics most kernels use, for IR text
// that carries no (template ...) of its own.  Spelled as the reference's registry
// spells them for CUDA-dialect targets (sarek/Sarek_stdlib/Float32.ml:41-157 and the
// Float64 / Int32 twins): a name with "%s" is a format, otherwise a function name.
const char *stdlib_template(const std::vector<std::string> &path, const std::string &n) {
  const std::string mod = path.empty() ? "" : path.back();
  const bool f32 = mod == "Float32", f64 = mod == "Float64";
  if (f32 || f64) {
    static const char *ops[][2] = {{"add", "(%s + %s)"}, {"minus", "(%s - %s)"}, {"sub", "(%s - %s)"},
                                   {"mul", "(%s * %s)"}, {"div", "(%s / %s)"}};
    for (auto &o : ops)
      if (n == o[0] || n == std::string(o[0]) + (f32 ? "_float32" : "_float64")) return o[1];
    static const char *fns[][3] = {
        {"sin", "sinf", "sin"}, {"cos", "cosf", "cos"}, {"tan", "tanf", "tan"},
        {"asin", "asinf", "asin"}, {"acos", "acosf", "acos"}, {"atan", "atanf", "atan"},
        {"sinh", "sinhf", "sinh"}, {"cosh", "coshf", "cosh"}, {"tanh", "tanhf", "tanh"},
        {"exp", "expf", "exp"}, {"log", "logf", "log"}, {"log10", "log10f", "log10"},
        {"sqrt", "sqrtf", "sqrt"}, {"ceil", "ceilf", "ceil"}, {"floor", "floorf", "floor"},
        {"expm1", "expm1f", "expm1"}, {"log1p", "log1pf", "log1p"}, {"abs_float", "fabsf", "fabs"},
        {"rsqrt", "rsqrtf", "rsqrt"}, {"pow", "powf", "pow"}, {"atan2", "atan2f", "atan2"},
        {"hypot", "hypotf", "hypot"}, {"copysign", "copysignf", "copysign"}};
    for (auto &f : fns)
      if (n == f[0]) return f32 ? f[1] : f[2];
    if (n == "of_int") return f32 ? "(float)(%s)" : "(double)(%s)";
    if (n == "to_int") return "(int)(%s)";
    if (f64 && n == "of_float32") return "(double)(%s)";
    if (f32 && n == "of_float64") return "(float)(%s)";
    // sarek/Sarek_float64/Float64.ml:133-146
    if (f64 && n == "of_int32") return "(double)(%s)";
    if (f64 && n == "to_int32") return "(int)(%s)";
    if (f64 && n == "to_float32") return "(float)(%s)";
  }
  if (mod == "Math") {   // sarek/Sarek_stdlib/Math.ml:19-35
    if (n == "xor") return "(%s ^ %s)";
    if (n == "logical_and") return "(%s & %s)";
    if (n == "pow") return "(int)powf((float)%s, (float)%s)";
  }
  if (mod == "Gpu" || mod == "Std") {   // sarek/Sarek_stdlib/Gpu.ml:117-247
    if (n == "float64_of_int") return "(double)(%s)";
    if (n == "int_of_float64") return "(int)(%s)";
    if (n == "spoc_powint") return "spoc_powint";
    if (n == "atomic_add_int32") return "atomicAdd(%s + %s, %s)";
    if (n == "atomic_inc_int32" || n == "atomic_inc_global_int32") return "atomicAdd(%s + %s, 1)";
  }
  const bool i32 = mod == "Int32", i64 = mod == "Int64";
  if (i32 || i64) {
    // sarek/Sarek_stdlib/Int32.ml:30-88 and Int64.ml:31-88
    static const char *ops[][2] = {{"add", "(%s + %s)"}, {"sub", "(%s - %s)"}, {"mul", "(%s * %s)"},
                                   {"div", "(%s / %s)"}, {"mod", "(%s %% %s)"}};
    for (auto &o : ops)
      if (n == o[0] || n == std::string(o[0]) + (i32 ? "_int32" : "_int64")) return o[1];
    static const char *same[][2] = {{"logand", "(%s & %s)"}, {"logor", "(%s | %s)"}, {"logxor", "(%s ^ %s)"},
                                    {"lognot", "(~%s)"}, {"shift_left", "(%s << %s)"}, {"shift_right", "(%s >> %s)"},
                                    {"neg", "(-%s)"}};
    for (auto &o : same)
      if (n == o[0]) return o[1];
    if (n == "shift_right_logical") return i32 ? "((unsigned int)%s >> %s)" : "((unsigned long)%s >> %s)";
    if (n == "abs") return i32 ? "abs(%s)" : "llabs(%s)";
    if (n == "of_float" || n == "of_int") return i32 ? "(int)(%s)" : "(long long)(%s)";
    if (n == "to_float") return "(double)(%s)";
    if (n == "to_int") return "(int)(%s)";
    if (i64 && n == "of_int32") return "(long long)(%s)";
    if (i64 && n == "to_int32") return "(int)(%s)";
  }
  if (n == "float" || n == "float_of_int") return "(float)(%s)";
  if (n == "int_of_float") return "(int)(%s)";
  return nullptr;
}

int count_placeholders(const std::string &t) {
  int c = 0;
  for (size_t i = 0; i + 1 < t.size(); ++i)
    if (t[i] == '%' && t[i + 1] == 's') {
      ++c;
      ++i;
    }
  return c;
}

std::string join_args(const std::vector<ExprP> &args) {
  std::string o;
  for (size_t i = 0; i < args.size(); ++i) o += (i ? ", " : "") + gen_expr(args[i]);
  return o;
}

std::string apply_template(const std::string &templ, const std::vector<ExprP> &args) {
  const int ph = count_placeholders(templ);
  if (ph == 0) return templ + "(" + join_args(args) + ")";
  if (ph != static_cast<int>(args.size()) || ph > 3) return templ + "(" + join_args(args) + ")";
  std::string o;
  size_t a = 0;
  for (size_t i = 0; i < templ.size(); ++i) {
    if (templ[i] == '%' && i + 1 < templ.size() && templ[i + 1] == 's') {
      const std::string arg = gen_expr(args[a++]);
      // "(-%s)" round "-5": a minus keeps a space from an operand that begins with one, here as in a negation
      if (!o.empty() && o.back() == '-' && !arg.empty() && arg[0] == '-') o.push_back(' ');
      o += arg;
      ++i;
    } else if (templ[i] == '%' && i + 1 < templ.size() && templ[i + 1] == '%') {
      o.push_back('%');   // the registry's templates are format strings: "%%" is the remainder operator
      ++i;
    } else {
      o.push_back(templ[i]);
    }
  }
  // The logical shifts are spelled with an unsigned operand (Int32.ml:68-72, Int64.ml:68-72), which leaves the whole
  // expression unsigned: `(x lsr 1) - 5 < 0` would never hold.  OCaml's result is the signed type again.
  if (templ == "((unsigned int)%s >> %s)") return "(int)" + o;
  if (templ == "((unsigned long)%s >> %s)") return "(long long)" + o;
  return o;
}

std::string atomic_call(const char *fn, const std::string &name, const std::vector<ExprP> &args,
                        bool allow_array_form) {
  if (args.size() == 2) return std::string(fn) + "(&" + gen_expr(args[0]) + ", " + gen_expr(args[1]) + ")";
  if (allow_array_form && args.size() == 3)
    return std::string(fn) + "(&" + gen_expr(args[0]) + "[" + gen_expr(args[1]) + "], " + gen_expr(args[2]) + ")";
  throw CodegenError("HIP codegen: intrinsic '" + name + "' called with " +
                     std::to_string(args.size()) + " arguments");
}

std::string gen_intrinsic(const Expr &e) {
  if (const char *t = thread_intrinsic(e.name)) return t;
  static const char *math1[] = {"sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh", "tanh",
                                "exp", "exp2", "log", "log2", "log10", "sqrt", "rsqrt", "cbrt",
                                "floor", "ceil", "round", "trunc", "fabs", "atan2", "pow", "fma",
                                "min", "max"};
  // Math names are emitted as plain calls whatever module they come from, as the
  // reference does (sarek-cuda/Sarek_ir_cuda.ml:268-292); HIP's overloads pick the f32
  // or f64 routine from the argument type.
  for (const char *m : math1)
    if (e.name == m) return e.name + "(" + join_args(e.args) + ")";
  if (e.name == "block_barrier") return "__syncthreads()";
  if (e.name == "atomic_add" || e.name == "atomic_add_int32" || e.name == "atomic_add_global_int32")
    return atomic_call("atomicAdd", e.name, e.args, true);
  if (e.name == "atomic_sub") return atomic_call("atomicSub", e.name, e.args, false);
  if (e.name == "atomic_min") return atomic_call("atomicMin", e.name, e.args, false);
  if (e.name == "atomic_max") return atomic_call("atomicMax", e.name, e.args, false);
  if (e.has_templ) return apply_template(e.templ, e.args);
  if (const char *t = stdlib_template(e.path, e.name)) return apply_template(t, e.args);
  std::string full;
  for (const auto &p : e.path) full += p + ".";
  return full + e.name + "(" + join_args(e.args) + ")";
}

const char *binop_str(Binop op) {
  static const char *s[] = {" + ", " - ", " * ", " / ", " % ", " == ", " != ", " < ", " <= ", " > ",
                            " >= ", " && ", " || ", " << ", " >> ", " & ", " | ", " ^ "};
  return s[static_cast<int>(op)];
}

// A floating constant: "%.17g" as the reference prints it (Sarek_ir_cuda.ml:83-89), which reads back as the same
// double.  Infinities and NaN come out of that format as "inf" / "nan", no C at all: they are written as the
// compiler's builtins, which need no header (the run-time compiler includes none that defines INFINITY or NAN).
std::string fmt17(double v, bool single) {
  char buf[64];
  if (std::isnan(v)) return single ? "__builtin_nanf(\"\")" : "__builtin_nan(\"\")";
  if (std::isinf(v)) {
    const char *inf = single ? "__builtin_inff()" : "__builtin_inf()";
    return v > 0 ? inf : std::string("(-") + inf + ")";
  }
  std::snprintf(buf, sizeof(buf), "%.17g", v);
  return buf;
}

std::string gen_lvalue(const LValueP &l) {
  switch (l->kind) {
    case LValue::LVar: return printed_name(l->var);
    case LValue::LArrayElem: return printed_name(l->name) + "[" + gen_expr(l->index) + "]";
    case LValue::LArrayElemExpr: return "(" + gen_expr(l->base) + ")[" + gen_expr(l->index) + "]";
    case LValue::LRecordField: return gen_lvalue(l->inner) + "." + l->name;
  }
  return "";
}

const std::vector<TypeP> *constructor_types(const std::string &cname) {
  if (!t_kernel) return nullptr;
  for (const auto &v : t_kernel->variants)
    for (const auto &c : v.second)
      if (c.first == cname) return &c.second;
  return nullptr;
}

std::string gen_match_case(const std::string &indent, const std::string &scrutinee,
                           const Pattern &p, const StmtP &body) {
  std::string o = indent;
  const bool names_the_value = !p.wildcard && p.constr.empty();   // `| x -> ...`
  if (p.wildcard || names_the_value) {
    o += "  default: {\n";
  } else {
    o += "  case " + p.constr + ": {\n";
  }
  CBlock braces;
  std::vector<std::unique_ptr<Binding>> bound;
  if (names_the_value) {
    // the reference prints `case : {` for it (Sarek_ir_cuda.ml:594-640 takes the empty name for a constructor)
    bound.push_back(std::make_unique<Binding>(p.vars.at(0)));
    o += indent + "    auto " + bound.back()->printed + " = " + scrutinee + ";\n";
  } else if (!p.wildcard) {
    const std::vector<TypeP> *types = constructor_types(p.constr);
    if (!p.vars.empty() && types && !types->empty()) {
      if (p.vars.size() == 1 && types->size() == 1) {
        bound.push_back(std::make_unique<Binding>(p.vars[0]));
        o += indent + "    " + type_str((*types)[0]) + " " + bound.back()->printed + " = " + scrutinee + ".data." +
             p.constr + "_v;\n";
      } else if (p.vars.size() == types->size()) {
        for (size_t i = 0; i < p.vars.size(); ++i) {
          bound.push_back(std::make_unique<Binding>(p.vars[i]));
          o += indent + "    " + type_str((*types)[i]) + " " + bound.back()->printed + " = " + scrutinee +
               ".data." + p.constr + "_v._" + std::to_string(i) + ";\n";
        }
      } else {
        throw CodegenError("HIP codegen: pattern '" + p.constr + "' binds " +
                           std::to_string(p.vars.size()) + " variables, constructor has " +
                           std::to_string(types->size()) + " arguments");
      }
    }
  }
  o += gen_stmt(body, indent + "    ");
  o += indent + "    break;\n" + indent + "  }\n";
  while (!bound.empty()) bound.pop_back();   // innermost first
  return o;
}

std::string gen_param(const Decl &d) {
  if (d.kind != Decl::Param) throw CodegenError("HIP codegen: local or shared declaration in the parameter list");
  std::string o = param_type_str(d.var.type) + " " + d.var.name;
  if (d.has_array_info || d.var.type->kind == Type::Vec) o += ", int sarek_" + d.var.name + "_length";
  return o;
}

std::string gen_local(const Decl &d, const std::string &indent) {
  switch (d.kind) {
    case Decl::Local:
      return indent + type_str(d.var.type) + " " + d.var.name +
             (d.init ? " = " + gen_expr(d.init) : "") + ";\n";
    case Decl::Shared:
      return indent + "__shared__ " + type_str(d.elt) + " " + d.name + "[" +
             (d.init ? gen_expr(d.init) : "") + "];\n";
    case Decl::Param: break;
  }
  throw CodegenError("HIP codegen: parameter declaration among the locals");
}

std::string gen_helper(const HelperFunc &f) {
  std::string o = "__device__ " + type_str(f.ret) + " " + f.name + "(";
  for (size_t i = 0; i < f.params.size(); ++i)
    o += (i ? ", " : "") + type_str(f.params[i].type) + " " + f.params[i].name;
  CBlock function;
  for (const auto &p : f.params) {
    t_c_blocks.back().push_back(p.name);
    t_renames.push_back({p.name, p.id, p.name, p.is_mutable});
  }
  o += ") {\n" + gen_stmt(f.body, "  ") + "}\n\n";
  return o;
}

std::string gen_variant_def(const std::string &name,
                            const std::vector<std::pair<std::string, std::vector<TypeP>>> &constrs) {
  const std::string m = mangle(name);
  std::string o = "enum { ";
  for (size_t i = 0; i < constrs.size(); ++i)
    o += (i ? ", " : "") + constrs[i].first + " = " + std::to_string(i);
  o += " };\ntypedef struct {\n  int tag;\n";
  bool payload = false;
  for (auto &c : constrs) payload |= !c.second.empty();
  if (payload) {
    o += "  union {\n";
    for (auto &c : constrs) {
      if (c.second.empty()) continue;
      if (c.second.size() == 1) {
        o += "    " + type_str(c.second[0]) + " " + c.first + "_v;\n";
      } else {
        o += "    struct { ";
        for (size_t i = 0; i < c.second.size(); ++i)
          o += (i ? " " : "") + type_str(c.second[i]) + " _" + std::to_string(i) + ";";
        o += " } " + c.first + "_v;\n";
      }
    }
    o += "  } data;\n";
  }
  o += "} " + m + ";\n\n";
  for (auto &c : constrs) {
    o += "__device__ __host__ inline " + m + " make_" + m + "_" + c.first + "(";
    if (c.second.size() == 1) {
      o += type_str(c.second[0]) + " v";
    } else {
      for (size_t j = 0; j < c.second.size(); ++j)
        o += (j ? ", " : "") + type_str(c.second[j]) + " v" + std::to_string(j);
    }
    o += ") {\n  " + m + " r;\n  r.tag = " + c.first + ";\n";
    if (c.second.size() == 1) {
      o += "  r.data." + c.first + "_v = v;\n";
    } else {
      for (size_t j = 0; j < c.second.size(); ++j)
        o += "  r.data." + c.first + "_v._" + std::to_string(j) + " = v" + std::to_string(j) + ";\n";
    }
    o += "  return r;\n}\n\n";
  }
  return o;
}

}  // namespace

std::string gen_expr(const ExprP &ep) {
  const Expr &e = *ep;
  switch (e.kind) {
    // The least value of a type has no literal of that type in C: 2147483648 is a long long and 9223372036854775808LL
    // does not fit, so "-2147483648" would make the arithmetic around it 64-bit.
    case Expr::ConstInt32:
      if (static_cast<int32_t>(e.ival) == INT32_MIN) return "(-2147483647 - 1)";
      return std::to_string(static_cast<int32_t>(e.ival));
    case Expr::ConstInt64:
      if (e.ival == INT64_MIN) return "(-9223372036854775807LL - 1)";
      return std::to_string(e.ival) + "LL";
    case Expr::ConstFloat32: {
      std::string s = fmt17(e.fval, true);
      if (std::isfinite(e.fval)) {
        if (s.find('.') == std::string::npos && s.find('e') == std::string::npos) s += ".0";
        s += "f";
      }
      return s;
    }
    case Expr::ConstFloat64: {
      // The reference prints "%.17g" as it is (Sarek_ir_cuda.ml:90), so 2.0 comes out as `2`, an int in C: `1.0 /. 2.0`
      // would be the integer division (1 / 2) and -0.0 the integer 0.  A whole value gets its decimal point here.
      std::string s = fmt17(e.fval, false);
      if (std::isfinite(e.fval) && s.find('.') == std::string::npos && s.find('e') == std::string::npos) s += ".0";
      return s;
    }
    case Expr::ConstBool: return e.ival ? "1" : "0";
    case Expr::ConstUnit: return "(void)0";
    case Expr::VarRef: return printed_name(e.var);
    case Expr::BinopE: return "(" + gen_expr(e.args[0]) + binop_str(e.binop) + gen_expr(e.args[1]) + ")";
    case Expr::UnopE: {
      // As the reference prints it, "(" op operand ")" -- except that the minus of a negation keeps a space from an
      // operand that itself begins with a minus (a negative literal): "(--3.5f)" is a decrement of a literal and does
      // not compile, there or here.
      const std::string operand = gen_expr(e.args[0]);
      const char *sign = e.unop == Unop::Neg ? (!operand.empty() && operand[0] == '-' ? "- " : "-")
                         : e.unop == Unop::Not ? "!" : "~";
      return std::string("(") + sign + operand + ")";
    }
    case Expr::ArrayRead: return printed_name(e.name) + "[" + gen_expr(e.args[0]) + "]";
    case Expr::ArrayReadExpr: return "(" + gen_expr(e.args[0]) + ")[" + gen_expr(e.args[1]) + "]";
    case Expr::RecordField: return gen_expr(e.args[0]) + "." + e.name;
    case Expr::Intrinsic: return gen_intrinsic(e);
    case Expr::Cast: return "(" + type_str(e.type) + ")" + gen_expr(e.args[0]);
    case Expr::Tuple: return "{" + join_args(e.args) + "}";
    case Expr::App: {
      if (e.args.empty()) throw CodegenError("HIP codegen: application without a function");
      std::vector<ExprP> rest(e.args.begin() + 1, e.args.end());
      return gen_expr(e.args[0]) + "(" + join_args(rest) + ")";
    }
    case Expr::Record: {
      std::string o = "(" + mangle(e.name) + "){";
      for (size_t i = 0; i < e.fields.size(); ++i) o += (i ? ", " : "") + gen_expr(e.fields[i].second);
      return o + "}";
    }
    case Expr::Variant:
      // A constructor without payload goes through its make_ function like the others.  (The reference prints the bare
      // tag there, sarek-cuda/Sarek_ir_cuda.ml:155: an enum constant where a value of the variant's struct type is
      // wanted, which no C++ compiler takes in `c = cond ? make_t_A(x) : B` or `t c = B`; none of its golden texts
      // has such a constructor.)
      return "make_" + mangle(e.name) + "_" + e.name2 + "(" + join_args(e.args) + ")";
    case Expr::ArrayLen: return "sarek_" + e.name + "_length";
    case Expr::ArrayCreate:
      throw CodegenError("HIP codegen: array creation is only valid as the value of a let binding");
    case Expr::If:
      return "(" + gen_expr(e.args[0]) + " ? " + gen_expr(e.args[1]) + " : " + gen_expr(e.args[2]) + ")";
    case Expr::Match: {
      // Nested conditionals on the tag, as the reference prints them (Sarek_ir_cuda.ml:179-208).  There a case's
      // variables stay undeclared (`match s with Circle r -> r *. r | ...` as a value does not compile); here each
      // stands for the payload it names, `s.data.Circle_v`, for the length of its case.
      if (e.cases.empty()) throw CodegenError("HIP codegen: empty match expression");
      const std::string scrutinee = gen_expr(e.args[0]);
      auto value_of = [&](const Pattern &p, const ExprP &body) {
        const size_t mark = t_renames.size();
        const std::vector<TypeP> *types =
            p.wildcard || p.vars.empty() || p.constr.empty() ? nullptr : constructor_types(p.constr);
        if (!p.wildcard && p.constr.empty() && p.vars.size() == 1)   // `| x -> ...`: x is the value itself
          t_renames.push_back({p.vars[0], -1, scrutinee, false});
        if (types && types->size() == p.vars.size())
          for (size_t i = 0; i < p.vars.size(); ++i)
            t_renames.push_back({p.vars[i], -1,
                                 scrutinee + ".data." + p.constr + "_v" +
                                     (p.vars.size() == 1 ? std::string() : "._" + std::to_string(i)),
                                 false});
        std::string text;
        try {
          text = gen_expr(body);
        } catch (...) {
          t_renames.erase(t_renames.begin() + static_cast<std::ptrdiff_t>(mark), t_renames.end());
          throw;
        }
        t_renames.erase(t_renames.begin() + static_cast<std::ptrdiff_t>(mark), t_renames.end());
        return text;
      };
      if (e.cases.size() == 1) return value_of(e.cases[0].first, e.cases[0].second);
      std::string o, close;
      for (size_t i = 0; i + 1 < e.cases.size(); ++i) {
        const Pattern &p = e.cases[i].first;
        o += "(" + (p.wildcard || p.constr.empty() ? std::string("1") : "(" + scrutinee + ".tag == " + p.constr + ")") + " ? " +
             value_of(p, e.cases[i].second) + " : ";
        close += ")";
      }
      return o + value_of(e.cases.back().first, e.cases.back().second) + close;
    }
  }
  return "";
}

// Whether nothing a loop's body does can change the expression's value: constants, immutable variables, the thread's
// indices and operators over those.
bool fixed_during_a_loop(const ExprP &ep) {
  if (!ep) return true;
  const Expr &e = *ep;
  switch (e.kind) {
    case Expr::ConstInt32: case Expr::ConstInt64: case Expr::ConstFloat32: case Expr::ConstFloat64:
    case Expr::ConstBool: case Expr::ConstUnit: case Expr::ArrayLen:
      return true;
    case Expr::VarRef: {
      const Rename *b = binding_of(e.var.name, e.var.id);
      return b ? !b->is_mutable : !e.var.is_mutable;
    }
    case Expr::Intrinsic:
      if (!e.args.empty() || !thread_intrinsic(e.name)) return false;
      return true;
    case Expr::BinopE: case Expr::UnopE: case Expr::Cast: case Expr::If: case Expr::RecordField:
      for (const auto &a : e.args)
        if (!fixed_during_a_loop(a)) return false;
      return true;
    default: return false;
  }
}

std::string gen_stmt(const StmtP &sp, const std::string &indent) {
  const Stmt &s = *sp;
  const std::string in2 = indent + "  ";
  switch (s.kind) {
    case Stmt::Empty: return "";
    case Stmt::Seq: {
      std::string o;
      for (const auto &c : s.stmts) o += gen_stmt(c, indent);
      return o;
    }
    case Stmt::Assign:
      if (s.e->kind == Expr::Record) {
        // Field by field, as the reference prints it (Sarek_ir_cuda.ml:440-444).  When a field's value reads the
        // record being assigned -- `p <- {x = p.y; y = p.x}` -- the later fields would see the earlier stores, where
        // OCaml builds the whole record first: the values are then taken into temporaries before the first store.
        const std::string target = gen_lvalue(s.lhs);
        std::string root;   // the variable or vector the target lives in; none for a computed base
        for (const LValue *l = s.lhs.get(); l;) {
          if (l->kind == LValue::LRecordField) {
            l = l->inner.get();
          } else {
            if (l->kind == LValue::LVar) root = printed_name(l->var);
            else if (l->kind == LValue::LArrayElem) root = printed_name(l->name);
            break;
          }
        }
        std::vector<std::string> values;
        bool reads_target = root.empty();
        for (const auto &f : s.e->fields) {
          values.push_back(gen_expr(f.second));
          for (size_t at = values.back().find(root); !reads_target && at != std::string::npos;
               at = values.back().find(root, at + 1)) {
            auto part_of_a_name = [](char c) { return std::isalnum(static_cast<unsigned char>(c)) || c == '_'; };
            const std::string &v = values.back();
            const bool starts = at == 0 || !part_of_a_name(v[at - 1]);
            const bool ends = at + root.size() >= v.size() || !part_of_a_name(v[at + root.size()]);
            reads_target = starts && ends;
          }
        }
        std::string o;
        if (!reads_target) {
          for (size_t i = 0; i < values.size(); ++i)
            o += indent + target + "." + s.e->fields[i].first + " = " + values[i] + ";\n";
          return o;
        }
        o = indent + "{\n";
        for (size_t i = 0; i < values.size(); ++i)
          o += in2 + "const auto sarek_field_" + std::to_string(i) + " = " + values[i] + ";\n";
        for (size_t i = 0; i < values.size(); ++i)
          o += in2 + target + "." + s.e->fields[i].first + " = sarek_field_" + std::to_string(i) + ";\n";
        return o + indent + "}\n";
      }
      return indent + gen_lvalue(s.lhs) + " = " + gen_expr(s.e) + ";\n";
    case Stmt::If: {
      std::string o = indent + "if (" + gen_expr(s.e) + ") {\n";
      {
        CBlock braces;
        o += gen_stmt(s.stmts[0], in2) + indent + "}";
      }
      if (s.stmts.size() > 1) {
        CBlock braces;
        o += " else {\n" + gen_stmt(s.stmts[1], in2) + indent + "}\n";
      } else {
        o += "\n";
      }
      return o;
    }
    case Stmt::While: {
      const std::string cond = gen_expr(s.e);
      CBlock braces;
      return indent + "while (" + cond + ") {\n" + gen_stmt(s.stmts[0], in2) + indent + "}\n";
    }
    case Stmt::For: {
      const char *op = s.downto ? ">=" : "<=";
      const char *inc = s.downto ? "--" : "++";
      const std::string from = gen_expr(s.e), to = gen_expr(s.e2);   // both with the outer meaning of the name
      CBlock scope;                                                  // the statement's own scope holds the counter
      Binding counter(s.var.name, s.var.id, false);
      // A bound that the body cannot change is printed in the condition, as the reference prints every bound
      // (Sarek_ir_cuda.ml:391-409).  One that reads a mutable variable, memory or a call would be evaluated again
      // in front of every turn there, where OCaml, the Native backend's loop and the reference's own walker
      // (Sarek_ir_interp.ml:858-872) evaluate it once: it is kept in a variable of the statement's scope.
      std::string stop = to, keep;
      std::unique_ptr<Binding> kept;
      if (!fixed_during_a_loop(s.e2)) {
        kept = std::make_unique<Binding>("sarek_to_" + counter.printed);
        stop = kept->printed;
        keep = ", " + stop + " = " + to;
      }
      CBlock braces;
      return indent + "for (" + type_str(s.var.type) + " " + counter.printed + " = " + from + keep + "; " +
             counter.printed + " " + op + " " + stop + "; " + counter.printed + inc + ") {\n" +
             gen_stmt(s.stmts[0], in2) + indent + "}\n";
    }
    case Stmt::Match: {
      const std::string scrutinee = gen_expr(s.e);
      std::string o = indent + "switch (" + scrutinee + ".tag) {\n";
      for (const auto &c : s.cases) o += gen_match_case(indent, scrutinee, c.first, c.second);
      return o + indent + "}\n";
    }
    case Stmt::Return: return indent + "return " + gen_expr(s.e) + ";\n";
    case Stmt::Barrier: return indent + "__syncthreads();\n";
    case Stmt::WarpBarrier: return indent + "__builtin_amdgcn_wave_barrier();\n";
    case Stmt::MemFence: return indent + "__threadfence();\n";
    case Stmt::Native: {
      std::string o = indent + s.native_code;
      if (s.native_code.empty() || s.native_code.back() != '\n') o += "\n";
      return o;
    }
    case Stmt::ExprS: return indent + gen_expr(s.e) + ";\n";
    case Stmt::Let:
    case Stmt::LetMut:
      if (s.kind == Stmt::Let && s.e->kind == Expr::ArrayCreate) {
        t_in_shared_size = s.e->mem == MemSpace::Shared;
        std::string size;
        try {
          size = gen_expr(s.e->args[0]);
        } catch (...) {
          t_in_shared_size = false;
          throw;
        }
        t_in_shared_size = false;
        Binding array(s.var);
        // An array a thread creates for itself starts at zero on the CPU backends (`Array.make size default`,
        // Sarek_native_gen.ml:466-469; the reference's IR walker likewise): `= {}` here, where the reference's text
        // leaves it uninitialised.  Shared arrays stay as declared: every kernel writes them before it reads.
        const bool shared = s.e->mem == MemSpace::Shared;
        return indent + (shared ? "__shared__ " : "") + type_str(s.e->type) + " " + array.printed + "[" + size + "]" +
               (shared ? "" : " = {}") + ";\n" + gen_stmt(s.stmts[0], indent);
      }
      if (s.var.type && s.var.type->kind == Type::Unit) {
        // `let () = e in body` (Sarek_lower_ir.ml:448-470 lowers it like any let): nothing to declare -- the
        // reference's `void u = e;` does not compile --, the value is evaluated for what it does
        return indent + gen_expr(s.e) + ";\n" + gen_stmt(s.stmts[0], indent);
      }
      {
        const std::string value = gen_expr(s.e);   // before the name changes its meaning
        Binding bound(s.var, s.kind == Stmt::LetMut);
        if (s.stmts[0]->kind == Stmt::Empty) bound.keep();
        return indent + type_str(s.var.type) + " " + bound.printed + " = " + value + ";\n" +
               gen_stmt(s.stmts[0], indent);
      }
    case Stmt::Pragma: {
      std::string o = indent + "#pragma ";
      for (size_t i = 0; i < s.hints.size(); ++i) o += (i ? " " : "") + s.hints[i];
      return o + "\n" + gen_stmt(s.stmts[0], indent);
    }
    case Stmt::Block: {
      CBlock braces;
      return indent + "{\n" + gen_stmt(s.stmts[0], in2) + indent + "}\n";
    }
  }
  return "";
}

FunctionScope::FunctionScope(const std::vector<std::string> &names) {
  t_c_blocks.clear();
  t_renames.clear();
  t_c_blocks.push_back(names);
}
FunctionScope::~FunctionScope() {
  t_c_blocks.clear();
  t_renames.clear();
}

std::string generate(const Kernel &k, const int block[3]) {
  for (int i = 0; i < 3; ++i) t_block[i] = block ? block[i] : 0;
  t_kernel = &k;
  t_c_blocks.clear();
  t_renames.clear();
  std::string o = "\nextern \"C\" {\n";
  try {
    // Type definitions: the variants, then the records, each in the order the kernel lists them (the reference's
    // order, sarek-cuda/Sarek_ir_cuda.ml:880-898) -- except that a type whose fields or payloads are of another of
    // the kernel's types waits until that one is defined (a record inside a record, a record as a variant's payload:
    // the reference's lists come out of a hash table and carry no such order).
    struct Def {
      bool is_variant;
      size_t index;
      const std::string *name;
    };
    std::vector<Def> defs;
    for (size_t i = 0; i < k.variants.size(); ++i) defs.push_back({true, i, &k.variants[i].first});
    for (size_t i = 0; i < k.types.size(); ++i) defs.push_back({false, i, &k.types[i].first});
    auto defined_here = [&](const std::string &n) {
      for (const Def &d : defs)
        if (*d.name == n) return true;
      return false;
    };
    auto needs = [&](const Def &d, const std::vector<bool> &done) {
      auto waits_for = [&](const TypeP &t) {
        if (!t || (t->kind != Type::Record && t->kind != Type::Variant) || t->name == *d.name || !defined_here(t->name))
          return false;
        for (size_t j = 0; j < defs.size(); ++j)
          if (*defs[j].name == t->name && !done[j]) return true;
        return false;
      };
      if (d.is_variant) {
        for (const auto &c : k.variants[d.index].second)
          for (const TypeP &t : c.second)
            if (waits_for(t)) return true;
      } else {
        for (const auto &f : k.types[d.index].second)
          if (waits_for(f.second)) return true;
      }
      return false;
    };
    std::vector<bool> done(defs.size(), false);
    for (size_t emitted = 0; emitted < defs.size(); ++emitted) {
      size_t pick = defs.size();
      for (size_t j = 0; j < defs.size() && pick == defs.size(); ++j)
        if (!done[j] && !needs(defs[j], done)) pick = j;
      if (pick == defs.size())   // types that contain each other: no order exists, the compiler will say so
        for (size_t j = 0; j < defs.size() && pick == defs.size(); ++j)
          if (!done[j]) pick = j;
      done[pick] = true;
      const Def &d = defs[pick];
      if (d.is_variant) {
        o += gen_variant_def(k.variants[d.index].first, k.variants[d.index].second);
      } else {
        const auto &t = k.types[d.index];
        o += "typedef struct {\n";
        for (const auto &f : t.second) o += "  " + type_str(f.second) + " " + f.first + ";\n";
        o += "} " + mangle(t.first) + ";\n\n";
      }
    }
    for (const auto &f : k.funcs) o += gen_helper(f);
    o += "__global__ void " + k.name + "(";
    for (size_t i = 0; i < k.params.size(); ++i) o += (i ? ", " : "") + gen_param(k.params[i]);
    o += ") {\n";
    CBlock function;
    for (const auto &d : k.params) {
      t_c_blocks.back().push_back(d.var.name);
      t_c_blocks.back().push_back("sarek_" + d.var.name + "_length");
      t_renames.push_back({d.var.name, d.var.id, d.var.name, d.var.is_mutable});
    }
    for (const auto &l : k.locals) {
      o += gen_local(l, "  ");
      t_c_blocks.back().push_back(l.kind == Decl::Shared ? l.name : l.var.name);
      if (l.kind != Decl::Shared) t_renames.push_back({l.var.name, l.var.id, l.var.name, true});
    }
    o += gen_stmt(k.body, "  ");
    o += "}\n}\n";
  } catch (...) {
    t_kernel = nullptr;
    throw;
  }
  t_kernel = nullptr;
  return o;
}

}  // namespace ir
}  // namespace sarek_hip
