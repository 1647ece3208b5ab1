// Text form of the kernel IR: reader and printer.
//
// The OCaml side of the plugin serialises a Sarek_ir_types.kernel value
// (spoc/ir/Sarek_ir_types.ml:230-245) into this s-expression form and hands it to
// sarek_hip_generate_source.  One form per constructor:
//
//   kernel  ::= (kernel NAME (params decl*) (locals decl*) (body stmt)
//                 [(types (NAME (FIELD type)*)*)] [(variants (NAME (CONSTR type*)*)*)]
//                 [(funcs (func NAME (params var*) type stmt)*)] [(native_fn true|false)])
//   decl    ::= (param var [(arr type memspace)]) | (local var [expr]) | (shared NAME type [expr])
//   var     ::= (var NAME ID type [mut])
//   type    ::= i32 | i64 | f32 | f64 | bool | unit | (vec type) | (array type memspace)
//             | (record NAME (FIELD type)*) | (variant NAME (CONSTR type*)*)
//   memspace::= global | shared | local
//   expr    ::= (i32 N) | (i64 N) | (f32 X) | (f64 X) | (bool true|false) | (unit) | var
//             | (OP expr expr)   OP = add sub mul div mod eq ne lt le gt ge and or shl shr
//                                     bitand bitor bitxor
//             | (neg e) | (not e) | (bitnot e) | (read NAME e) | (readx e e) | (field e NAME)
//             | (intr (PATH*) NAME [(template "TEXT")] e*) | (cast type e) | (tuple e*)
//             | (app e e*) | (record NAME (FIELD e)*) | (variant TYPE CONSTR e*) | (len NAME)
//             | (newarray type e memspace) | (if e e e) | (match e (case pat e)*)
//   pat     ::= _ | (CONSTR VAR*)
//   lvalue  ::= (lvar var) | (lelem NAME e) | (lelemx e e) | (lfield lvalue NAME)
//   stmt    ::= (assign lvalue e) | (seq stmt*) | (if e stmt [stmt]) | (while e stmt)
//             | (for var e e upto|downto stmt) | (match e (case pat stmt)*) | (return e)
//             | (barrier) | (warpbarrier) | (memfence) | (expr e) | (empty)
//             | (let var e stmt) | (letmut var e stmt) | (pragma (HINT*) stmt) | (block stmt)
//             | (native "CODE")
//
// `(template ...)` carries the device-code template the caller's intrinsic registry holds
// for a non-builtin intrinsic (Sarek_registry.fun_device_template,
// spoc/registry/Sarek_registry.ml:167-197); `(native ...)` carries the text an SNative
// node produces for this backend.  Floating constants are written with enough digits to
// round-trip (OCaml "%.17g"); nan, inf and -inf are accepted.
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <sstream>

#include "ir.hpp"

namespace sarek_hip {
namespace ir {
namespace {

struct SExp {
  bool atom = false, quoted = false;
  std::string text;
  std::vector<SExp> items;
  size_t pos = 0;
};

[[noreturn]] void perr(const SExp &at, const std::string &msg) {
  throw ParseError("IR text, offset " + std::to_string(at.pos) + ": " + msg);
}

class Reader {
 public:
  static constexpr int kMaxDepth = 2000;
  explicit Reader(const std::string &s) : s_(s) {}
  SExp read_all() {
    SExp e = read();
    skip();
    if (i_ != s_.size()) throw ParseError("IR text: trailing characters at offset " + std::to_string(i_));
    return e;
  }

 private:
  void skip() {
    while (i_ < s_.size()) {
      if (std::isspace(static_cast<unsigned char>(s_[i_]))) {
        ++i_;
      } else if (s_[i_] == ';') {
        while (i_ < s_.size() && s_[i_] != '\n') ++i_;
      } else {
        break;
      }
    }
  }
  SExp read() {
    skip();
    if (i_ >= s_.size()) throw ParseError("IR text: unexpected end of input");
    SExp e;
    e.pos = i_;
    if (s_[i_] == '(') {
      ++i_;
      // every later pass recurses over this tree: bound its depth here, far above any
      // real kernel, so that no input can run the caller's stack out
      if (++depth_ > kMaxDepth)
        throw ParseError("IR text: nesting deeper than " + std::to_string(kMaxDepth) + " at offset " +
                         std::to_string(e.pos));
      for (;;) {
        skip();
        if (i_ >= s_.size()) throw ParseError("IR text: unbalanced '(' opened at offset " + std::to_string(e.pos));
        if (s_[i_] == ')') {
          ++i_;
          --depth_;
          return e;
        }
        e.items.push_back(read());
      }
    }
    if (s_[i_] == ')') throw ParseError("IR text: unexpected ')' at offset " + std::to_string(i_));
    e.atom = true;
    if (s_[i_] == '"') {
      e.quoted = true;
      ++i_;
      while (i_ < s_.size() && s_[i_] != '"') {
        if (s_[i_] == '\\' && i_ + 1 < s_.size()) {
          ++i_;
          char c = s_[i_];
          e.text.push_back(c == 'n' ? '\n' : c == 't' ? '\t' : c);
        } else {
          e.text.push_back(s_[i_]);
        }
        ++i_;
      }
      if (i_ >= s_.size()) throw ParseError("IR text: unterminated string at offset " + std::to_string(e.pos));
      ++i_;
      return e;
    }
    while (i_ < s_.size() && !std::isspace(static_cast<unsigned char>(s_[i_])) && s_[i_] != '(' &&
           s_[i_] != ')')
      e.text.push_back(s_[i_++]);
    return e;
  }
  const std::string &s_;
  size_t i_ = 0;
  int depth_ = 0;
};

const std::string &head(const SExp &e) {
  if (e.atom || e.items.empty() || !e.items[0].atom) perr(e, "expected a form (HEAD ...)");
  return e.items[0].text;
}

const std::string &atom(const SExp &e, const char *what) {
  if (!e.atom) perr(e, std::string("expected ") + what);
  return e.text;
}

void arity(const SExp &e, size_t lo, size_t hi) {
  const size_t n = e.items.size() - 1;
  if (n < lo || n > hi)
    perr(e, "form '" + head(e) + "' takes " + std::to_string(lo) +
                (hi == lo ? "" : ".." + (hi == SIZE_MAX ? std::string("*") : std::to_string(hi))) +
                " arguments, got " + std::to_string(n));
}

MemSpace to_mem(const SExp &e) {
  const std::string &a = atom(e, "a memory space");
  if (a == "global") return MemSpace::Global;
  if (a == "shared") return MemSpace::Shared;
  if (a == "local") return MemSpace::Local;
  perr(e, "unknown memory space '" + a + "'");
}

TypeP to_type(const SExp &e) {
  auto t = std::make_shared<Type>();
  if (e.atom) {
    const std::string &a = e.text;
    if (a == "i32") t->kind = Type::Int32;
    else if (a == "i64") t->kind = Type::Int64;
    else if (a == "f32") t->kind = Type::Float32;
    else if (a == "f64") t->kind = Type::Float64;
    else if (a == "bool") t->kind = Type::Bool;
    else if (a == "unit") t->kind = Type::Unit;
    else perr(e, "unknown type '" + a + "'");
    return t;
  }
  const std::string &h = head(e);
  if (h == "vec") {
    arity(e, 1, 1);
    t->kind = Type::Vec;
    t->elt = to_type(e.items[1]);
  } else if (h == "array") {
    arity(e, 2, 2);
    t->kind = Type::Array;
    t->elt = to_type(e.items[1]);
    t->mem = to_mem(e.items[2]);
  } else if (h == "record") {
    arity(e, 1, SIZE_MAX);
    t->kind = Type::Record;
    t->name = atom(e.items[1], "a record name");
    for (size_t i = 2; i < e.items.size(); ++i) {
      const SExp &f = e.items[i];
      if (f.atom || f.items.size() != 2) perr(f, "expected (FIELD type)");
      t->fields.emplace_back(atom(f.items[0], "a field name"), to_type(f.items[1]));
    }
  } else if (h == "variant") {
    arity(e, 1, SIZE_MAX);
    t->kind = Type::Variant;
    t->name = atom(e.items[1], "a variant name");
    for (size_t i = 2; i < e.items.size(); ++i) {
      const SExp &c = e.items[i];
      if (c.atom || c.items.empty()) perr(c, "expected (CONSTR type*)");
      std::vector<TypeP> args;
      for (size_t j = 1; j < c.items.size(); ++j) args.push_back(to_type(c.items[j]));
      t->constrs.emplace_back(atom(c.items[0], "a constructor name"), args);
    }
  } else {
    perr(e, "unknown type form '" + h + "'");
  }
  return t;
}

Var to_var(const SExp &e) {
  if (e.atom || head(e) != "var") perr(e, "expected (var NAME ID type [mut])");
  arity(e, 3, 4);
  Var v;
  v.name = atom(e.items[1], "a variable name");
  v.id = std::atoi(atom(e.items[2], "a variable id").c_str());
  v.type = to_type(e.items[3]);
  if (e.items.size() == 5) {
    if (atom(e.items[4], "'mut'") != "mut") perr(e.items[4], "expected 'mut'");
    v.is_mutable = true;
  }
  return v;
}

int64_t to_int(const SExp &e) {
  const std::string &a = atom(e, "an integer");
  char *end = nullptr;
  long long v = std::strtoll(a.c_str(), &end, 10);
  if (end == a.c_str() || *end) perr(e, "malformed integer '" + a + "'");
  return v;
}

double to_float(const SExp &e) {
  const std::string &a = atom(e, "a floating constant");
  if (a == "nan") return std::nan("");
  if (a == "inf" || a == "infinity") return INFINITY;
  if (a == "-inf" || a == "neg_infinity") return -INFINITY;
  char *end = nullptr;
  double v = std::strtod(a.c_str(), &end);
  if (end == a.c_str() || *end) perr(e, "malformed floating constant '" + a + "'");
  return v;
}

Pattern to_pattern(const SExp &e) {
  Pattern p;
  if (e.atom) {
    if (e.text != "_") perr(e, "expected _ or (CONSTR VAR*)");
    return p;
  }
  if (e.items.empty()) perr(e, "empty pattern");
  p.wildcard = false;
  p.constr = atom(e.items[0], "a constructor name");
  for (size_t i = 1; i < e.items.size(); ++i) p.vars.push_back(atom(e.items[i], "a variable name"));
  // `| x -> ...`: the front end lowers a variable pattern to a constructor pattern with an empty name and the one
  // variable (Sarek_lower_ir.ml:556-559); written (? x) here
  if (p.constr == "?") {
    if (p.vars.size() != 1) perr(e, "expected (? VAR)");
    p.constr.clear();
  }
  return p;
}

const struct {
  const char *name;
  Binop op;
} kBinops[] = {{"add", Binop::Add}, {"sub", Binop::Sub}, {"mul", Binop::Mul}, {"div", Binop::Div},
               {"mod", Binop::Mod}, {"eq", Binop::Eq}, {"ne", Binop::Ne}, {"lt", Binop::Lt},
               {"le", Binop::Le}, {"gt", Binop::Gt}, {"ge", Binop::Ge}, {"and", Binop::And},
               {"or", Binop::Or}, {"shl", Binop::Shl}, {"shr", Binop::Shr},
               {"bitand", Binop::BitAnd}, {"bitor", Binop::BitOr}, {"bitxor", Binop::BitXor}};

ExprP to_expr(const SExp &e) {
  auto x = std::make_shared<Expr>();
  const std::string &h = head(e);
  for (const auto &b : kBinops)
    if (h == b.name) {
      arity(e, 2, 2);
      x->kind = Expr::BinopE;
      x->binop = b.op;
      x->args = {to_expr(e.items[1]), to_expr(e.items[2])};
      return x;
    }
  if (h == "i32" || h == "i64") {
    arity(e, 1, 1);
    x->kind = h == "i32" ? Expr::ConstInt32 : Expr::ConstInt64;
    x->ival = to_int(e.items[1]);
  } else if (h == "f32" || h == "f64") {
    arity(e, 1, 1);
    x->kind = h == "f32" ? Expr::ConstFloat32 : Expr::ConstFloat64;
    x->fval = to_float(e.items[1]);
  } else if (h == "bool") {
    arity(e, 1, 1);
    x->kind = Expr::ConstBool;
    const std::string &a = atom(e.items[1], "true or false");
    if (a != "true" && a != "false") perr(e.items[1], "expected true or false");
    x->ival = a == "true";
  } else if (h == "unit") {
    arity(e, 0, 0);
    x->kind = Expr::ConstUnit;
  } else if (h == "var") {
    x->kind = Expr::VarRef;
    x->var = to_var(e);
  } else if (h == "neg" || h == "not" || h == "bitnot") {
    arity(e, 1, 1);
    x->kind = Expr::UnopE;
    x->unop = h == "neg" ? Unop::Neg : h == "not" ? Unop::Not : Unop::BitNot;
    x->args = {to_expr(e.items[1])};
  } else if (h == "read") {
    arity(e, 2, 2);
    x->kind = Expr::ArrayRead;
    x->name = atom(e.items[1], "an array name");
    x->args = {to_expr(e.items[2])};
  } else if (h == "readx") {
    arity(e, 2, 2);
    x->kind = Expr::ArrayReadExpr;
    x->args = {to_expr(e.items[1]), to_expr(e.items[2])};
  } else if (h == "field") {
    arity(e, 2, 2);
    x->kind = Expr::RecordField;
    x->args = {to_expr(e.items[1])};
    x->name = atom(e.items[2], "a field name");
  } else if (h == "intr") {
    arity(e, 2, SIZE_MAX);
    x->kind = Expr::Intrinsic;
    const SExp &p = e.items[1];
    if (p.atom) perr(p, "expected a module path list");
    for (const auto &c : p.items) x->path.push_back(atom(c, "a module name"));
    x->name = atom(e.items[2], "an intrinsic name");
    size_t i = 3;
    if (i < e.items.size() && !e.items[i].atom && !e.items[i].items.empty() &&
        e.items[i].items[0].atom && e.items[i].items[0].text == "template") {
      if (e.items[i].items.size() != 2) perr(e.items[i], "expected (template \"TEXT\")");
      x->templ = atom(e.items[i].items[1], "a template string");
      x->has_templ = true;
      ++i;
    }
    for (; i < e.items.size(); ++i) x->args.push_back(to_expr(e.items[i]));
  } else if (h == "cast") {
    arity(e, 2, 2);
    x->kind = Expr::Cast;
    x->type = to_type(e.items[1]);
    x->args = {to_expr(e.items[2])};
  } else if (h == "tuple") {
    x->kind = Expr::Tuple;
    for (size_t i = 1; i < e.items.size(); ++i) x->args.push_back(to_expr(e.items[i]));
  } else if (h == "app") {
    arity(e, 1, SIZE_MAX);
    x->kind = Expr::App;
    for (size_t i = 1; i < e.items.size(); ++i) x->args.push_back(to_expr(e.items[i]));
  } else if (h == "record") {
    arity(e, 1, SIZE_MAX);
    x->kind = Expr::Record;
    x->name = atom(e.items[1], "a record type name");
    for (size_t i = 2; i < e.items.size(); ++i) {
      const SExp &f = e.items[i];
      if (f.atom || f.items.size() != 2) perr(f, "expected (FIELD expr)");
      x->fields.emplace_back(atom(f.items[0], "a field name"), to_expr(f.items[1]));
    }
  } else if (h == "variant") {
    arity(e, 2, SIZE_MAX);
    x->kind = Expr::Variant;
    x->name = atom(e.items[1], "a variant type name");
    x->name2 = atom(e.items[2], "a constructor name");
    for (size_t i = 3; i < e.items.size(); ++i) x->args.push_back(to_expr(e.items[i]));
  } else if (h == "len") {
    arity(e, 1, 1);
    x->kind = Expr::ArrayLen;
    x->name = atom(e.items[1], "an array name");
  } else if (h == "newarray") {
    arity(e, 3, 3);
    x->kind = Expr::ArrayCreate;
    x->type = to_type(e.items[1]);
    x->args = {to_expr(e.items[2])};
    x->mem = to_mem(e.items[3]);
  } else if (h == "if") {
    arity(e, 3, 3);
    x->kind = Expr::If;
    x->args = {to_expr(e.items[1]), to_expr(e.items[2]), to_expr(e.items[3])};
  } else if (h == "match") {
    arity(e, 1, SIZE_MAX);
    x->kind = Expr::Match;
    x->args = {to_expr(e.items[1])};
    for (size_t i = 2; i < e.items.size(); ++i) {
      const SExp &c = e.items[i];
      if (c.atom || c.items.size() != 3 || head(c) != "case") perr(c, "expected (case pat expr)");
      x->cases.emplace_back(to_pattern(c.items[1]), to_expr(c.items[2]));
    }
  } else {
    perr(e, "unknown expression form '" + h + "'");
  }
  return x;
}

LValueP to_lvalue(const SExp &e) {
  auto l = std::make_shared<LValue>();
  const std::string &h = head(e);
  if (h == "lvar") {
    arity(e, 1, 1);
    l->kind = LValue::LVar;
    l->var = to_var(e.items[1]);
  } else if (h == "lelem") {
    arity(e, 2, 2);
    l->kind = LValue::LArrayElem;
    l->name = atom(e.items[1], "an array name");
    l->index = to_expr(e.items[2]);
  } else if (h == "lelemx") {
    arity(e, 2, 2);
    l->kind = LValue::LArrayElemExpr;
    l->base = to_expr(e.items[1]);
    l->index = to_expr(e.items[2]);
  } else if (h == "lfield") {
    arity(e, 2, 2);
    l->kind = LValue::LRecordField;
    l->inner = to_lvalue(e.items[1]);
    l->name = atom(e.items[2], "a field name");
  } else {
    perr(e, "unknown lvalue form '" + h + "'");
  }
  return l;
}

StmtP to_stmt(const SExp &e) {
  auto s = std::make_shared<Stmt>();
  const std::string &h = head(e);
  if (h == "assign") {
    arity(e, 2, 2);
    s->kind = Stmt::Assign;
    s->lhs = to_lvalue(e.items[1]);
    s->e = to_expr(e.items[2]);
  } else if (h == "seq") {
    s->kind = Stmt::Seq;
    for (size_t i = 1; i < e.items.size(); ++i) s->stmts.push_back(to_stmt(e.items[i]));
  } else if (h == "if") {
    arity(e, 2, 3);
    s->kind = Stmt::If;
    s->e = to_expr(e.items[1]);
    s->stmts.push_back(to_stmt(e.items[2]));
    if (e.items.size() == 4) s->stmts.push_back(to_stmt(e.items[3]));
  } else if (h == "while") {
    arity(e, 2, 2);
    s->kind = Stmt::While;
    s->e = to_expr(e.items[1]);
    s->stmts = {to_stmt(e.items[2])};
  } else if (h == "for") {
    arity(e, 5, 5);
    s->kind = Stmt::For;
    s->var = to_var(e.items[1]);
    s->e = to_expr(e.items[2]);
    s->e2 = to_expr(e.items[3]);
    const std::string &d = atom(e.items[4], "upto or downto");
    if (d != "upto" && d != "downto") perr(e.items[4], "expected upto or downto");
    s->downto = d == "downto";
    s->stmts = {to_stmt(e.items[5])};
  } else if (h == "match") {
    arity(e, 1, SIZE_MAX);
    s->kind = Stmt::Match;
    s->e = to_expr(e.items[1]);
    for (size_t i = 2; i < e.items.size(); ++i) {
      const SExp &c = e.items[i];
      if (c.atom || c.items.size() != 3 || head(c) != "case") perr(c, "expected (case pat stmt)");
      s->cases.emplace_back(to_pattern(c.items[1]), to_stmt(c.items[2]));
    }
  } else if (h == "return") {
    arity(e, 1, 1);
    s->kind = Stmt::Return;
    s->e = to_expr(e.items[1]);
  } else if (h == "barrier") {
    s->kind = Stmt::Barrier;
  } else if (h == "warpbarrier") {
    s->kind = Stmt::WarpBarrier;
  } else if (h == "memfence") {
    s->kind = Stmt::MemFence;
  } else if (h == "expr") {
    arity(e, 1, 1);
    s->kind = Stmt::ExprS;
    s->e = to_expr(e.items[1]);
  } else if (h == "empty") {
    s->kind = Stmt::Empty;
  } else if (h == "let" || h == "letmut") {
    arity(e, 3, 3);
    s->kind = h == "let" ? Stmt::Let : Stmt::LetMut;
    s->var = to_var(e.items[1]);
    s->e = to_expr(e.items[2]);
    s->stmts = {to_stmt(e.items[3])};
  } else if (h == "pragma") {
    arity(e, 2, 2);
    s->kind = Stmt::Pragma;
    if (e.items[1].atom) perr(e.items[1], "expected a list of pragma words");
    for (const auto &w : e.items[1].items) s->hints.push_back(atom(w, "a pragma word"));
    s->stmts = {to_stmt(e.items[2])};
  } else if (h == "block") {
    arity(e, 1, 1);
    s->kind = Stmt::Block;
    s->stmts = {to_stmt(e.items[1])};
  } else if (h == "native") {
    arity(e, 1, 1);
    s->kind = Stmt::Native;
    s->native_code = atom(e.items[1], "a code string");
  } else {
    perr(e, "unknown statement form '" + h + "'");
  }
  return s;
}

Decl to_decl(const SExp &e) {
  Decl d;
  const std::string &h = head(e);
  if (h == "param") {
    arity(e, 1, 2);
    d.kind = Decl::Param;
    d.var = to_var(e.items[1]);
    if (e.items.size() == 3) {
      const SExp &a = e.items[2];
      if (a.atom || a.items.size() != 3 || head(a) != "arr") perr(a, "expected (arr type memspace)");
      d.has_array_info = true;
      d.arr_elt = to_type(a.items[1]);
      d.arr_mem = to_mem(a.items[2]);
    }
  } else if (h == "local") {
    arity(e, 1, 2);
    d.kind = Decl::Local;
    d.var = to_var(e.items[1]);
    if (e.items.size() == 3) d.init = to_expr(e.items[2]);
  } else if (h == "shared") {
    arity(e, 2, 3);
    d.kind = Decl::Shared;
    d.name = atom(e.items[1], "a shared array name");
    d.elt = to_type(e.items[2]);
    if (e.items.size() == 4) d.init = to_expr(e.items[3]);
  } else {
    perr(e, "unknown declaration form '" + h + "'");
  }
  return d;
}

Kernel to_kernel(const SExp &e) {
  if (e.atom || head(e) != "kernel") perr(e, "expected (kernel NAME ...)");
  if (e.items.size() < 2) perr(e, "kernel without a name");
  Kernel k;
  k.name = atom(e.items[1], "a kernel name");
  bool have_body = false;
  for (size_t i = 2; i < e.items.size(); ++i) {
    const SExp &sec = e.items[i];
    const std::string &h = head(sec);
    if (h == "params") {
      for (size_t j = 1; j < sec.items.size(); ++j) {
        // any declaration, as kern_params : decl list; the lowering rejects what is not a parameter
        k.params.push_back(to_decl(sec.items[j]));
      }
    } else if (h == "locals") {
      for (size_t j = 1; j < sec.items.size(); ++j) {
        Decl d = to_decl(sec.items[j]);
        if (d.kind == Decl::Param) perr(sec.items[j], "(param ...) is not allowed in (locals ...)");
        k.locals.push_back(d);
      }
    } else if (h == "body") {
      arity(sec, 1, 1);
      k.body = to_stmt(sec.items[1]);
      have_body = true;
    } else if (h == "types") {
      for (size_t j = 1; j < sec.items.size(); ++j) {
        const SExp &t = sec.items[j];
        if (t.atom || t.items.empty()) perr(t, "expected (NAME (FIELD type)*)");
        std::vector<std::pair<std::string, TypeP>> fields;
        for (size_t f = 1; f < t.items.size(); ++f) {
          if (t.items[f].atom || t.items[f].items.size() != 2) perr(t.items[f], "expected (FIELD type)");
          fields.emplace_back(atom(t.items[f].items[0], "a field name"), to_type(t.items[f].items[1]));
        }
        k.types.emplace_back(atom(t.items[0], "a record name"), fields);
      }
    } else if (h == "variants") {
      for (size_t j = 1; j < sec.items.size(); ++j) {
        const SExp &t = sec.items[j];
        if (t.atom || t.items.empty()) perr(t, "expected (NAME (CONSTR type*)*)");
        std::vector<std::pair<std::string, std::vector<TypeP>>> cs;
        for (size_t c = 1; c < t.items.size(); ++c) {
          const SExp &ce = t.items[c];
          if (ce.atom || ce.items.empty()) perr(ce, "expected (CONSTR type*)");
          std::vector<TypeP> args;
          for (size_t a = 1; a < ce.items.size(); ++a) args.push_back(to_type(ce.items[a]));
          cs.emplace_back(atom(ce.items[0], "a constructor name"), args);
        }
        k.variants.emplace_back(atom(t.items[0], "a variant name"), cs);
      }
    } else if (h == "funcs") {
      for (size_t j = 1; j < sec.items.size(); ++j) {
        const SExp &f = sec.items[j];
        if (f.atom || f.items.size() != 5 || head(f) != "func")
          perr(f, "expected (func NAME (params var*) type stmt)");
        HelperFunc hf;
        hf.name = atom(f.items[1], "a function name");
        if (f.items[2].atom || head(f.items[2]) != "params") perr(f.items[2], "expected (params var*)");
        for (size_t p = 1; p < f.items[2].items.size(); ++p) hf.params.push_back(to_var(f.items[2].items[p]));
        hf.ret = to_type(f.items[3]);
        hf.body = to_stmt(f.items[4]);
        k.funcs.push_back(hf);
      }
    } else if (h == "native_fn") {
      arity(sec, 1, 1);
      k.has_native_fn = atom(sec.items[1], "true or false") == "true";
    } else {
      perr(sec, "unknown kernel section '" + h + "'");
    }
  }
  if (!have_body) perr(e, "kernel without a (body ...)");
  return k;
}

// ---- printer --------------------------------------------------------------------
std::string fmt_float(double v) {
  if (std::isnan(v)) return "nan";
  if (std::isinf(v)) return v > 0 ? "inf" : "-inf";
  char buf[64];
  std::snprintf(buf, sizeof(buf), "%.17g", v);
  return buf;
}

const char *mem_name(MemSpace m) {
  return m == MemSpace::Global ? "global" : m == MemSpace::Shared ? "shared" : "local";
}

std::string quote(const std::string &s) {
  std::string o = "\"";
  for (char c : s) {
    if (c == '"' || c == '\\') o.push_back('\\');
    if (c == '\n') {
      o += "\\n";
      continue;
    }
    o.push_back(c);
  }
  return o + "\"";
}

std::string pr_type(const TypeP &t) {
  switch (t->kind) {
    case Type::Int32: return "i32";
    case Type::Int64: return "i64";
    case Type::Float32: return "f32";
    case Type::Float64: return "f64";
    case Type::Bool: return "bool";
    case Type::Unit: return "unit";
    case Type::Vec: return "(vec " + pr_type(t->elt) + ")";
    case Type::Array: return "(array " + pr_type(t->elt) + " " + mem_name(t->mem) + ")";
    case Type::Record: {
      std::string s = "(record " + t->name;
      for (auto &f : t->fields) s += " (" + f.first + " " + pr_type(f.second) + ")";
      return s + ")";
    }
    case Type::Variant: {
      std::string s = "(variant " + t->name;
      for (auto &c : t->constrs) {
        s += " (" + c.first;
        for (auto &a : c.second) s += " " + pr_type(a);
        s += ")";
      }
      return s + ")";
    }
  }
  return "unit";
}

std::string pr_var(const Var &v) {
  return "(var " + v.name + " " + std::to_string(v.id) + " " + pr_type(v.type) +
         (v.is_mutable ? " mut)" : ")");
}

std::string pr_pat(const Pattern &p) {
  if (p.wildcard) return "_";
  std::string s = "(" + (p.constr.empty() ? std::string("?") : p.constr);
  for (auto &v : p.vars) s += " " + v;
  return s + ")";
}

std::string pr_expr(const ExprP &e) {
  switch (e->kind) {
    case Expr::ConstInt32: return "(i32 " + std::to_string(e->ival) + ")";
    case Expr::ConstInt64: return "(i64 " + std::to_string(e->ival) + ")";
    case Expr::ConstFloat32: return "(f32 " + fmt_float(e->fval) + ")";
    case Expr::ConstFloat64: return "(f64 " + fmt_float(e->fval) + ")";
    case Expr::ConstBool: return e->ival ? "(bool true)" : "(bool false)";
    case Expr::ConstUnit: return "(unit)";
    case Expr::VarRef: return pr_var(e->var);
    case Expr::BinopE:
      return std::string("(") + kBinops[static_cast<int>(e->binop)].name + " " + pr_expr(e->args[0]) +
             " " + pr_expr(e->args[1]) + ")";
    case Expr::UnopE:
      return std::string("(") + (e->unop == Unop::Neg ? "neg" : e->unop == Unop::Not ? "not" : "bitnot") +
             " " + pr_expr(e->args[0]) + ")";
    case Expr::ArrayRead: return "(read " + e->name + " " + pr_expr(e->args[0]) + ")";
    case Expr::ArrayReadExpr: return "(readx " + pr_expr(e->args[0]) + " " + pr_expr(e->args[1]) + ")";
    case Expr::RecordField: return "(field " + pr_expr(e->args[0]) + " " + e->name + ")";
    case Expr::Intrinsic: {
      std::string s = "(intr (";
      for (size_t i = 0; i < e->path.size(); ++i) s += (i ? " " : "") + e->path[i];
      s += ") " + e->name;
      if (e->has_templ) s += " (template " + quote(e->templ) + ")";
      for (auto &a : e->args) s += " " + pr_expr(a);
      return s + ")";
    }
    case Expr::Cast: return "(cast " + pr_type(e->type) + " " + pr_expr(e->args[0]) + ")";
    case Expr::Tuple:
    case Expr::App: {
      std::string s = e->kind == Expr::Tuple ? "(tuple" : "(app";
      for (auto &a : e->args) s += " " + pr_expr(a);
      return s + ")";
    }
    case Expr::Record: {
      std::string s = "(record " + e->name;
      for (auto &f : e->fields) s += " (" + f.first + " " + pr_expr(f.second) + ")";
      return s + ")";
    }
    case Expr::Variant: {
      std::string s = "(variant " + e->name + " " + e->name2;
      for (auto &a : e->args) s += " " + pr_expr(a);
      return s + ")";
    }
    case Expr::ArrayLen: return "(len " + e->name + ")";
    case Expr::ArrayCreate:
      return "(newarray " + pr_type(e->type) + " " + pr_expr(e->args[0]) + " " + mem_name(e->mem) + ")";
    case Expr::If:
      return "(if " + pr_expr(e->args[0]) + " " + pr_expr(e->args[1]) + " " + pr_expr(e->args[2]) + ")";
    case Expr::Match: {
      std::string s = "(match " + pr_expr(e->args[0]);
      for (auto &c : e->cases) s += " (case " + pr_pat(c.first) + " " + pr_expr(c.second) + ")";
      return s + ")";
    }
  }
  return "(unit)";
}

std::string pr_lvalue(const LValueP &l) {
  switch (l->kind) {
    case LValue::LVar: return "(lvar " + pr_var(l->var) + ")";
    case LValue::LArrayElem: return "(lelem " + l->name + " " + pr_expr(l->index) + ")";
    case LValue::LArrayElemExpr: return "(lelemx " + pr_expr(l->base) + " " + pr_expr(l->index) + ")";
    case LValue::LRecordField: return "(lfield " + pr_lvalue(l->inner) + " " + l->name + ")";
  }
  return "";
}

std::string pr_stmt(const StmtP &s, const std::string &ind) {
  const std::string in2 = ind + "  ";
  switch (s->kind) {
    case Stmt::Assign: return ind + "(assign " + pr_lvalue(s->lhs) + " " + pr_expr(s->e) + ")";
    case Stmt::Seq: {
      std::string o = ind + "(seq";
      for (auto &c : s->stmts) o += "\n" + pr_stmt(c, in2);
      return o + ")";
    }
    case Stmt::If: {
      std::string o = ind + "(if " + pr_expr(s->e) + "\n" + pr_stmt(s->stmts[0], in2);
      if (s->stmts.size() > 1) o += "\n" + pr_stmt(s->stmts[1], in2);
      return o + ")";
    }
    case Stmt::While: return ind + "(while " + pr_expr(s->e) + "\n" + pr_stmt(s->stmts[0], in2) + ")";
    case Stmt::For:
      return ind + "(for " + pr_var(s->var) + " " + pr_expr(s->e) + " " + pr_expr(s->e2) +
             (s->downto ? " downto\n" : " upto\n") + pr_stmt(s->stmts[0], in2) + ")";
    case Stmt::Match: {
      std::string o = ind + "(match " + pr_expr(s->e);
      for (auto &c : s->cases) o += "\n" + in2 + "(case " + pr_pat(c.first) + "\n" + pr_stmt(c.second, in2 + "  ") + ")";
      return o + ")";
    }
    case Stmt::Return: return ind + "(return " + pr_expr(s->e) + ")";
    case Stmt::Barrier: return ind + "(barrier)";
    case Stmt::WarpBarrier: return ind + "(warpbarrier)";
    case Stmt::MemFence: return ind + "(memfence)";
    case Stmt::ExprS: return ind + "(expr " + pr_expr(s->e) + ")";
    case Stmt::Empty: return ind + "(empty)";
    case Stmt::Let:
    case Stmt::LetMut:
      return ind + (s->kind == Stmt::Let ? "(let " : "(letmut ") + pr_var(s->var) + " " + pr_expr(s->e) +
             "\n" + pr_stmt(s->stmts[0], in2) + ")";
    case Stmt::Pragma: {
      std::string o = ind + "(pragma (";
      for (size_t i = 0; i < s->hints.size(); ++i) o += (i ? " " : "") + s->hints[i];
      return o + ")\n" + pr_stmt(s->stmts[0], in2) + ")";
    }
    case Stmt::Block: return ind + "(block\n" + pr_stmt(s->stmts[0], in2) + ")";
    case Stmt::Native: return ind + "(native " + quote(s->native_code) + ")";
  }
  return ind + "(empty)";
}

std::string pr_decl(const Decl &d) {
  switch (d.kind) {
    case Decl::Param:
      return "(param " + pr_var(d.var) +
             (d.has_array_info ? " (arr " + pr_type(d.arr_elt) + " " + mem_name(d.arr_mem) + "))" : ")");
    case Decl::Local: return "(local " + pr_var(d.var) + (d.init ? " " + pr_expr(d.init) : "") + ")";
    case Decl::Shared:
      return "(shared " + d.name + " " + pr_type(d.elt) + (d.init ? " " + pr_expr(d.init) : "") + ")";
  }
  return "";
}

}  // namespace

Kernel parse_kernel(const std::string &text) { return to_kernel(Reader(text).read_all()); }
StmtP parse_stmt(const std::string &text) { return to_stmt(Reader(text).read_all()); }
ExprP parse_expr(const std::string &text) { return to_expr(Reader(text).read_all()); }
std::string print_expr(const ExprP &e) { return pr_expr(e); }
std::string print_stmt(const StmtP &s) { return pr_stmt(s, ""); }

std::string print_kernel(const Kernel &k) {
  std::string o = "(kernel " + k.name + "\n  (params";
  for (auto &p : k.params) o += "\n    " + pr_decl(p);
  o += ")\n  (locals";
  for (auto &l : k.locals) o += "\n    " + pr_decl(l);
  o += ")\n  (body\n" + pr_stmt(k.body, "    ") + ")";
  if (!k.types.empty()) {
    o += "\n  (types";
    for (auto &t : k.types) {
      o += " (" + t.first;
      for (auto &f : t.second) o += " (" + f.first + " " + pr_type(f.second) + ")";
      o += ")";
    }
    o += ")";
  }
  if (!k.variants.empty()) {
    o += "\n  (variants";
    for (auto &v : k.variants) {
      o += " (" + v.first;
      for (auto &c : v.second) {
        o += " (" + c.first;
        for (auto &a : c.second) o += " " + pr_type(a);
        o += ")";
      }
      o += ")";
    }
    o += ")";
  }
  if (!k.funcs.empty()) {
    o += "\n  (funcs";
    for (auto &f : k.funcs) {
      o += "\n    (func " + f.name + " (params";
      for (auto &p : f.params) o += " " + pr_var(p);
      o += ") " + pr_type(f.ret) + "\n" + pr_stmt(f.body, "      ") + ")";
    }
    o += ")";
  }
  o += std::string("\n  (native_fn ") + (k.has_native_fn ? "true" : "false") + "))\n";
  return o;
}

}  // namespace ir
}  // namespace sarek_hip
