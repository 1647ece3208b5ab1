// Kernel fusion on the IR (sarek/sarek/Sarek_fusion.ml), restated over the C++ IR.
//
// Results are meant to equal the reference's on the same kernels, its blind spots
// included: expressions the reference's structural equality does not look into (casts,
// record fields, ...) never compare equal, writes through computed array expressions are
// not collected, a conditional producer write is not inlined, and the map -> reduce
// rewrite inserts the producer's expression as it stands (still indexed by the producer's
// own index expression, not by the reduction's loop variable).
#include "fusion.hpp"

#include <algorithm>
#include <cstdlib>

namespace sarek_hip {
namespace ir {
namespace fusion {
namespace {

using Access = std::pair<std::string, ExprP>;   // (array, index expression)

bool is_const(const ExprP &e) { return e->kind <= Expr::ConstUnit; }

// Copy of `e` with every direct child expression replaced by f(child).
template <class F>
ExprP with_children(const ExprP &e, F f) {
  auto n = std::make_shared<Expr>(*e);
  for (auto &a : n->args) a = f(a);
  for (auto &fl : n->fields) fl.second = f(fl.second);
  for (auto &c : n->cases) c.second = f(c.second);
  return n;
}

template <class F>
bool any_child(const ExprP &e, F f) {
  for (auto &a : e->args)
    if (f(a)) return true;
  for (auto &fl : e->fields)
    if (f(fl.second)) return true;
  for (auto &c : e->cases)
    if (f(c.second)) return true;
  return false;
}

ExprP int32_const(int v) {
  auto c = std::make_shared<Expr>();
  c->kind = Expr::ConstInt32;
  c->ival = v;
  return c;
}

ExprP binop(Binop op, const ExprP &a, const ExprP &b) {
  auto n = std::make_shared<Expr>();
  n->kind = Expr::BinopE;
  n->binop = op;
  n->args = {a, b};
  return n;
}

// Reads of an expression, appended in evaluation order; the reference conses each read in
// front of what its sub-expressions and earlier siblings produced, so its list is this
// vector reversed (Sarek_fusion.ml:198-223).
void reads_of_expr(std::vector<Access> &acc, const ExprP &e) {
  switch (e->kind) {
    case Expr::ArrayRead:
      reads_of_expr(acc, e->args[0]);
      acc.emplace_back(e->name, e->args[0]);
      return;
    case Expr::ArrayLen:
    case Expr::ArrayCreate:
    case Expr::VarRef:
      return;
    default:
      if (is_const(e)) return;
      for (auto &a : e->args) reads_of_expr(acc, a);
      for (auto &f : e->fields) reads_of_expr(acc, f.second);
      for (auto &c : e->cases) reads_of_expr(acc, c.second);
  }
}

void writes_of_stmt(std::vector<Access> &acc, const StmtP &s) {
  switch (s->kind) {
    case Stmt::Assign:
      if (s->lhs->kind == LValue::LArrayElem) acc.emplace_back(s->lhs->name, s->lhs->index);
      return;
    case Stmt::Match:
      for (auto &c : s->cases) writes_of_stmt(acc, c.second);
      return;
    case Stmt::Seq: case Stmt::If: case Stmt::While: case Stmt::For: case Stmt::Let: case Stmt::LetMut:
    case Stmt::Pragma: case Stmt::Block:
      for (auto &b : s->stmts) writes_of_stmt(acc, b);
      return;
    default:
      return;
  }
}

void reads_of_stmt(std::vector<Access> &acc, const StmtP &s) {
  switch (s->kind) {
    case Stmt::Assign:
      if (s->lhs->kind == LValue::LArrayElem) reads_of_expr(acc, s->lhs->index);
      reads_of_expr(acc, s->e);
      return;
    case Stmt::Seq: case Stmt::Pragma: case Stmt::Block:
      for (auto &b : s->stmts) reads_of_stmt(acc, b);
      return;
    case Stmt::If: case Stmt::While: case Stmt::Let: case Stmt::LetMut:
      reads_of_expr(acc, s->e);
      for (auto &b : s->stmts) reads_of_stmt(acc, b);
      return;
    case Stmt::For:
      reads_of_expr(acc, s->e);
      reads_of_expr(acc, s->e2);
      reads_of_stmt(acc, s->stmts[0]);
      return;
    case Stmt::Match:
      reads_of_expr(acc, s->e);
      for (auto &c : s->cases) reads_of_stmt(acc, c.second);
      return;
    case Stmt::Return: case Stmt::ExprS:
      reads_of_expr(acc, s->e);
      return;
    default:
      return;
  }
}

// The reference's lists: most recent first.
std::vector<Access> read_list(const StmtP &body) {
  std::vector<Access> v;
  reads_of_stmt(v, body);
  std::reverse(v.begin(), v.end());
  return v;
}
std::vector<Access> write_list(const StmtP &body) {
  std::vector<Access> v;
  writes_of_stmt(v, body);
  std::reverse(v.begin(), v.end());
  return v;
}

// idx = base + const | base - const | const + base  (Sarek_fusion.ml:284-289)
bool extract_offset(const ExprP &idx, ExprP &base, int &off) {
  if (idx->kind != Expr::BinopE) return false;
  const ExprP &l = idx->args[0], &r = idx->args[1];
  if (idx->binop == Binop::Add && r->kind == Expr::ConstInt32) {
    base = l;
    off = static_cast<int>(r->ival);
    return true;
  }
  if (idx->binop == Binop::Sub && r->kind == Expr::ConstInt32) {
    base = l;
    off = -static_cast<int>(r->ival);
    return true;
  }
  if (idx->binop == Binop::Add && l->kind == Expr::ConstInt32) {
    base = r;
    off = static_cast<int>(l->ival);
    return true;
  }
  return false;
}

bool is_base_index(const ExprP &idx) { return idx->kind == Expr::VarRef || idx->kind == Expr::Intrinsic; }

AccessPattern analyze_pattern(const std::vector<Access> &accesses, const std::string &arr) {
  std::vector<ExprP> mine;
  for (auto &a : accesses)
    if (a.first == arr) mine.push_back(a.second);
  AccessPattern p;
  if (mine.empty()) return p;   // Unknown
  if (mine.size() == 1) {
    p.kind = AccessPattern::OneToOne;
    p.index = mine[0];
    return p;
  }
  p.kind = AccessPattern::Gather;
  std::vector<std::pair<ExprP, int>> based;
  for (auto &idx : mine) {
    ExprP base;
    int off = 0;
    if (extract_offset(idx, base, off)) based.emplace_back(base, off);
    else if (is_base_index(idx)) based.emplace_back(idx, 0);
  }
  if (based.size() != mine.size()) return p;
  for (size_t i = 1; i < based.size(); ++i)
    if (!expr_equal(based[i].first, based[0].first)) return p;
  p.kind = AccessPattern::Stencil;
  for (auto &b : based) p.offsets.push_back(b.second);
  std::sort(p.offsets.begin(), p.offsets.end());
  p.offsets.erase(std::unique(p.offsets.begin(), p.offsets.end()), p.offsets.end());
  return p;
}

const AccessPattern *find(const std::vector<std::pair<std::string, AccessPattern>> &l, const std::string &arr) {
  for (auto &p : l)
    if (p.first == arr) return &p.second;
  return nullptr;
}

bool contains(const std::vector<std::string> &l, const std::string &x) {
  return std::find(l.begin(), l.end(), x) != l.end();
}

std::vector<std::string> names_of(const std::vector<std::pair<std::string, AccessPattern>> &l) {
  std::vector<std::string> n;
  for (auto &p : l) n.push_back(p.first);
  return n;
}

// The expression a kernel stores to arr[idx], when that store is unconditional
// (Sarek_fusion.ml:360-378).
ExprP find_write_expr(const StmtP &s, const std::string &arr, const ExprP &idx) {
  switch (s->kind) {
    case Stmt::Assign:
      if (s->lhs->kind == LValue::LArrayElem && s->lhs->name == arr && expr_equal(s->lhs->index, idx)) return s->e;
      return nullptr;
    case Stmt::Seq:
      for (auto &b : s->stmts)
        if (ExprP e = find_write_expr(b, arr, idx)) return e;
      return nullptr;
    case Stmt::Let: case Stmt::LetMut: case Stmt::Pragma: case Stmt::Block:
      return find_write_expr(s->stmts[0], arr, idx);
    default:
      return nullptr;
  }
}

const std::string *decl_name(const Decl &d) {
  if (d.kind == Decl::Param) return &d.var.name;
  if (d.kind == Decl::Shared) return &d.name;
  return nullptr;
}

template <class T>
std::vector<T> concat(const std::vector<T> &a, const std::vector<T> &b) {
  std::vector<T> r = a;
  r.insert(r.end(), b.begin(), b.end());
  return r;
}

// Consumer with `body`, without the intermediate, plus what the producer brings along
// (Sarek_fusion.ml:490-547, 713-757, 976-1019).
Kernel merged(const Kernel &producer, const Kernel &consumer, const std::string &intermediate,
              const StmtP &body, const char *suffix) {
  Kernel k;
  k.name = consumer.name + suffix;
  std::vector<std::string> kept;
  for (auto &d : consumer.params) {
    const std::string *n = decl_name(d);
    if (n && *n == intermediate) continue;
    k.params.push_back(d);
    if (n) kept.push_back(*n);
  }
  for (auto &d : producer.params) {
    const std::string *n = decl_name(d);
    if (n && (*n == intermediate || contains(kept, *n))) continue;
    k.params.push_back(d);
  }
  k.locals = concat(consumer.locals, producer.locals);
  k.body = body;
  k.types = concat(consumer.types, producer.types);
  k.variants = concat(consumer.variants, producer.variants);
  k.funcs = concat(consumer.funcs, producer.funcs);
  k.has_native_fn = false;
  return k;
}

ExprP shift_expr(const ExprP &e, int offset) {
  if (offset == 0) return e;
  switch (e->kind) {
    case Expr::ArrayRead: {
      auto n = std::make_shared<Expr>(*e);
      n->args[0] = offset > 0 ? binop(Binop::Add, e->args[0], int32_const(offset))
                              : binop(Binop::Sub, e->args[0], int32_const(-offset));
      return n;
    }
    case Expr::BinopE: case Expr::UnopE: case Expr::Intrinsic: case Expr::Cast: case Expr::Tuple:
      return with_children(e, [&](const ExprP &c) { return shift_expr(c, offset); });
    default:
      return e;
  }
}

ExprP subst_stencil_reads(const std::string &arr, const ExprP &base_idx, const ExprP &producer_expr,
                          int offset_shift, const ExprP &e) {
  switch (e->kind) {
    case Expr::ArrayRead: {
      if (e->name != arr) return e;
      ExprP base;
      int off = 0;
      if (extract_offset(e->args[0], base, off))
        return expr_equal(base, base_idx) ? shift_expr(producer_expr, off + offset_shift) : e;
      return expr_equal(e->args[0], base_idx) ? shift_expr(producer_expr, offset_shift) : e;
    }
    case Expr::BinopE: case Expr::UnopE: case Expr::Intrinsic: case Expr::Cast: case Expr::Tuple:
      return with_children(
          e, [&](const ExprP &c) { return subst_stencil_reads(arr, base_idx, producer_expr, offset_shift, c); });
    default:
      return e;
  }
}

template <class F>
StmtP with_bodies(const StmtP &s, F f) {
  auto n = std::make_shared<Stmt>(*s);
  for (auto &b : n->stmts) b = f(b);
  for (auto &c : n->cases) c.second = f(c.second);
  return n;
}

}  // namespace

const char *binop_name(Binop op) {
  static const char *const names[] = {"add", "sub", "mul", "div", "mod", "eq", "ne", "lt", "le",
                                      "gt", "ge", "and", "or", "shl", "shr", "bitand", "bitor", "bitxor"};
  return names[static_cast<int>(op)];
}

// Sarek_fusion.ml:35-48: constants, variables (by id), operators, named-array reads and
// intrinsics are compared; any other form is unequal to everything, itself included.
bool expr_equal(const ExprP &a, const ExprP &b) {
  if (is_const(a) && is_const(b)) {
    if (a->kind != b->kind) return false;
    if (a->kind == Expr::ConstFloat32 || a->kind == Expr::ConstFloat64) return a->fval == b->fval;
    return a->kind == Expr::ConstUnit || a->ival == b->ival;
  }
  if (a->kind != b->kind) return false;
  switch (a->kind) {
    case Expr::VarRef: return a->var.id == b->var.id;
    case Expr::BinopE:
      return a->binop == b->binop && expr_equal(a->args[0], b->args[0]) && expr_equal(a->args[1], b->args[1]);
    case Expr::UnopE: return a->unop == b->unop && expr_equal(a->args[0], b->args[0]);
    case Expr::ArrayRead: return a->name == b->name && expr_equal(a->args[0], b->args[0]);
    case Expr::Intrinsic:
      if (a->path != b->path || a->name != b->name || a->args.size() != b->args.size()) return false;
      for (size_t i = 0; i < a->args.size(); ++i)
        if (!expr_equal(a->args[i], b->args[i])) return false;
      return true;
    default: return false;
  }
}

bool expr_uses_array(const std::string &arr, const ExprP &e) {
  switch (e->kind) {
    case Expr::ArrayRead: return e->name == arr || expr_uses_array(arr, e->args[0]);
    case Expr::ArrayLen: case Expr::ArrayCreate: case Expr::VarRef: return false;
    default:
      return !is_const(e) && any_child(e, [&](const ExprP &c) { return expr_uses_array(arr, c); });
  }
}

ExprP subst_array_read(const std::string &arr, const ExprP &idx, const ExprP &replacement, const ExprP &e) {
  switch (e->kind) {
    case Expr::ArrayRead:
      if (e->name == arr && expr_equal(e->args[0], idx)) return replacement;
      break;
    case Expr::ArrayLen: case Expr::ArrayCreate: case Expr::VarRef: return e;
    default:
      if (is_const(e)) return e;
  }
  return with_children(e, [&](const ExprP &c) { return subst_array_read(arr, idx, replacement, c); });
}

StmtP subst_array_read_stmt(const std::string &arr, const ExprP &idx, const ExprP &replacement, const StmtP &s) {
  auto on_expr = [&](const ExprP &e) { return subst_array_read(arr, idx, replacement, e); };
  switch (s->kind) {
    case Stmt::Barrier: case Stmt::WarpBarrier: case Stmt::MemFence: case Stmt::Empty: case Stmt::Native:
      return s;
    default:
      break;
  }
  auto n = std::make_shared<Stmt>(*with_bodies(
      s, [&](const StmtP &b) { return subst_array_read_stmt(arr, idx, replacement, b); }));
  if (n->e) n->e = on_expr(n->e);
  if (n->e2) n->e2 = on_expr(n->e2);
  if (s->kind == Stmt::Assign && s->lhs->kind == LValue::LArrayElem) {
    auto lv = std::make_shared<LValue>(*s->lhs);
    lv->index = on_expr(lv->index);
    n->lhs = lv;
  }
  return n;
}

bool stmt_uses_array(const std::string &arr, const StmtP &s) {
  auto in_expr = [&](const ExprP &e) { return e && expr_uses_array(arr, e); };
  if (s->kind == Stmt::Assign && s->lhs->kind == LValue::LArrayElem &&
      (s->lhs->name == arr || in_expr(s->lhs->index)))
    return true;
  switch (s->kind) {
    case Stmt::Barrier: case Stmt::WarpBarrier: case Stmt::MemFence: case Stmt::Empty: case Stmt::Native:
      return false;
    default:
      break;
  }
  if (in_expr(s->e) || in_expr(s->e2)) return true;
  for (auto &b : s->stmts)
    if (stmt_uses_array(arr, b)) return true;
  for (auto &c : s->cases)
    if (stmt_uses_array(arr, c.second)) return true;
  return false;
}

bool has_barrier(const StmtP &s) {
  if (s->kind == Stmt::Barrier || s->kind == Stmt::WarpBarrier) return true;
  for (auto &b : s->stmts)
    if (has_barrier(b)) return true;
  for (auto &c : s->cases)
    if (has_barrier(c.second)) return true;
  return false;
}

Info analyze(const Kernel &k) {
  const std::vector<Access> reads = read_list(k.body), writes = write_list(k.body);
  auto by_array = [](const std::vector<Access> &l) {
    std::vector<std::string> names;
    for (auto &a : l) names.push_back(a.first);
    std::sort(names.begin(), names.end());
    names.erase(std::unique(names.begin(), names.end()), names.end());
    std::vector<std::pair<std::string, AccessPattern>> out;
    for (auto &n : names) out.emplace_back(n, analyze_pattern(l, n));
    return out;
  };
  Info info;
  info.reads = by_array(reads);
  info.writes = by_array(writes);
  info.has_barriers = has_barrier(k.body);
  info.has_atomics = false;   // the reference does not detect atomics either
  return info;
}

bool can_fuse(const Kernel &producer, const Kernel &consumer, const std::string &intermediate) {
  const Info p = analyze(producer), c = analyze(consumer);
  const AccessPattern *w = find(p.writes, intermediate), *r = find(c.reads, intermediate);
  return w && r && w->kind == AccessPattern::OneToOne && r->kind == AccessPattern::OneToOne &&
         !p.has_barriers && !c.has_barriers;
}

Kernel fuse(const Kernel &producer, const Kernel &consumer, const std::string &intermediate) {
  ExprP idx;
  for (auto &a : read_list(consumer.body))
    if (a.first == intermediate) {
      idx = a.second;
      break;
    }
  if (!idx) return consumer;
  const ExprP replacement = find_write_expr(producer.body, intermediate, idx);
  if (!replacement) return consumer;
  return merged(producer, consumer, intermediate,
                subst_array_read_stmt(intermediate, idx, replacement, consumer.body), "_fused");
}

std::pair<Kernel, std::vector<std::string>> fuse_pipeline(const std::vector<Kernel> &kernels) {
  if (kernels.empty()) throw EmptyPipeline("fuse_pipeline: cannot fuse empty kernel list");
  Kernel current = kernels[0];
  std::vector<std::string> eliminated;
  for (size_t i = 1; i < kernels.size(); ++i) {
    const Kernel &k = kernels[i];
    const std::vector<std::string> writes = names_of(analyze(current).writes), reads = names_of(analyze(k).reads);
    const std::string *inter = nullptr;
    for (auto &w : writes)
      if (contains(reads, w)) {
        inter = &w;
        break;
      }
    if (inter && can_fuse(current, k, *inter)) {
      eliminated.insert(eliminated.begin(), *inter);
      current = fuse(current, k, *inter);
    } else {
      current = k;
    }
  }
  return {current, eliminated};
}

std::optional<ReductionLoop> detect_reduction_pattern(const StmtP &s) {
  if (s->kind != Stmt::For || s->downto) return std::nullopt;
  const StmtP &body = s->stmts[0];
  if (body->kind != Stmt::Assign || body->lhs->kind != LValue::LVar || body->e->kind != Expr::BinopE)
    return std::nullopt;
  const Var &acc = body->lhs->var;
  for (int flip = 0; flip < 2; ++flip) {
    const ExprP &a = body->e->args[flip], &r = body->e->args[1 - flip];
    if (a->kind == Expr::VarRef && a->var.id == acc.id && r->kind == Expr::ArrayRead &&
        r->args[0]->kind == Expr::VarRef && r->args[0]->var.id == s->var.id)
      return ReductionLoop{acc, body->e->binop, r->name, s->var};
  }
  return std::nullopt;
}

std::optional<Binop> is_reduction_kernel(const Kernel &k, const std::string &arr) {
  struct Finder {
    const std::string &arr;
    std::optional<Binop> operator()(const StmtP &s) const {
      if (s->kind == Stmt::Seq) {
        for (auto &b : s->stmts)
          if (auto r = (*this)(b)) return r;
        return std::nullopt;
      }
      auto r = detect_reduction_pattern(s);
      if (r && r->array == arr) return r->op;
      return std::nullopt;
    }
  };
  return Finder{arr}(k.body);
}

bool can_fuse_reduction(const Kernel &map, const Kernel &reduce, const std::string &intermediate) {
  const Info m = analyze(map), r = analyze(reduce);
  const AccessPattern *w = find(m.writes, intermediate);
  return w && w->kind == AccessPattern::OneToOne && is_reduction_kernel(reduce, intermediate).has_value() &&
         !m.has_barriers && !r.has_barriers;
}

Kernel fuse_reduction(const Kernel &map, const Kernel &reduce, const std::string &intermediate) {
  ExprP idx;
  for (auto &a : write_list(map.body))
    if (a.first == intermediate) {
      idx = a.second;
      break;
    }
  if (!idx) return reduce;
  const ExprP replacement = find_write_expr(map.body, intermediate, idx);
  if (!replacement) return reduce;
  struct Rewriter {
    const std::string &intermediate;
    const ExprP &replacement;
    StmtP operator()(const StmtP &s) const {
      switch (s->kind) {
        case Stmt::For: {
          auto loop = detect_reduction_pattern(s);
          auto n = std::make_shared<Stmt>(*s);
          if (loop && loop->array == intermediate) {
            auto loop_index = std::make_shared<Expr>();
            loop_index->kind = Expr::VarRef;
            loop_index->var = s->var;
            n->stmts[0] = subst_array_read_stmt(intermediate, loop_index, replacement, s->stmts[0]);
          } else {
            n->stmts[0] = (*this)(s->stmts[0]);
          }
          return n;
        }
        case Stmt::Seq: case Stmt::If: case Stmt::While: case Stmt::Match:
          return with_bodies(s, *this);
        default:
          return s;
      }
    }
  };
  return merged(map, reduce, intermediate, Rewriter{intermediate, replacement}(reduce.body), "_fused");
}

std::optional<Kernel> try_fuse(const Kernel &producer, const Kernel &consumer, const std::string &intermediate) {
  if (can_fuse_reduction(producer, consumer, intermediate)) return fuse_reduction(producer, consumer, intermediate);
  if (can_fuse(producer, consumer, intermediate)) return fuse(producer, consumer, intermediate);
  return std::nullopt;
}

int stencil_radius(const std::vector<int> &offsets) {
  int r = 0;
  for (int o : offsets) r = std::max(r, std::abs(o));
  return r;
}

std::optional<std::vector<int>> get_stencil_info(const Kernel &k, const std::string &arr) {
  const Info info = analyze(k);
  const AccessPattern *p = find(info.reads, arr);
  if (p && p->kind == AccessPattern::Stencil) return p->offsets;
  if (p && p->kind == AccessPattern::OneToOne) return std::vector<int>{0};
  return std::nullopt;
}

bool can_fuse_stencil(const Kernel &producer, const Kernel &consumer, const std::string &intermediate) {
  const Info p = analyze(producer), c = analyze(consumer);
  const AccessPattern *r = find(c.reads, intermediate);
  return find(p.writes, intermediate) && r &&
         (r->kind == AccessPattern::Stencil || r->kind == AccessPattern::OneToOne) && !p.has_barriers &&
         !c.has_barriers;
}

std::optional<StencilFusionInfo> analyze_stencil_fusion(const Kernel &producer, const Kernel &consumer,
                                                        const std::string &intermediate) {
  const Info p = analyze(producer), c = analyze(consumer);
  StencilFusionInfo out;
  for (auto &r : p.reads)
    if (r.first != intermediate && r.second.kind == AccessPattern::Stencil)
      out.producer_radius = std::max(out.producer_radius, stencil_radius(r.second.offsets));
  const AccessPattern *r = find(c.reads, intermediate);
  if (r && r->kind == AccessPattern::Stencil) out.consumer_radius = stencil_radius(r->offsets);
  else if (r && r->kind == AccessPattern::OneToOne) out.consumer_radius = 0;
  else return std::nullopt;
  for (auto &rd : p.reads)
    if (rd.first != intermediate) out.input_arrays.push_back(rd.first);
  out.combined_radius = out.producer_radius + out.consumer_radius;
  return out;
}

Kernel fuse_stencil(const Kernel &producer, const Kernel &consumer, const std::string &intermediate) {
  ExprP write_idx;
  for (auto &a : write_list(producer.body))
    if (a.first == intermediate) {
      write_idx = a.second;
      break;
    }
  if (!write_idx) return consumer;
  const ExprP replacement = find_write_expr(producer.body, intermediate, write_idx);
  if (!replacement) return consumer;
  struct Rewriter {
    const std::string &intermediate;
    const ExprP &write_idx, &replacement;
    ExprP on_expr(const ExprP &e) const { return subst_stencil_reads(intermediate, write_idx, replacement, 0, e); }
    StmtP operator()(const StmtP &s) const {
      switch (s->kind) {
        case Stmt::Assign: {
          auto n = std::make_shared<Stmt>(*s);
          n->e = on_expr(s->e);
          return n;
        }
        case Stmt::If: case Stmt::While: case Stmt::Match: {
          auto n = std::make_shared<Stmt>(*with_bodies(s, *this));
          n->e = on_expr(s->e);
          return n;
        }
        case Stmt::Seq: case Stmt::For:
          return with_bodies(s, *this);
        default:
          return s;
      }
    }
  };
  return merged(producer, consumer, intermediate, Rewriter{intermediate, write_idx, replacement}(consumer.body),
                "_stencil_fused");
}

std::optional<Kernel> try_fuse_all(const Kernel &producer, const Kernel &consumer,
                                   const std::string &intermediate) {
  if (can_fuse_reduction(producer, consumer, intermediate)) return fuse_reduction(producer, consumer, intermediate);
  if (can_fuse_stencil(producer, consumer, intermediate)) return fuse_stencil(producer, consumer, intermediate);
  if (can_fuse(producer, consumer, intermediate)) return fuse(producer, consumer, intermediate);
  return std::nullopt;
}

Hint should_fuse(const Kernel &producer, const Kernel &consumer, const std::string &intermediate) {
  const Info p = analyze(producer), c = analyze(consumer);
  if (p.has_barriers || c.has_barriers) return {Decision::DontFuse, "Barrier prevents fusion"};
  const AccessPattern *w = find(p.writes, intermediate), *r = find(c.reads, intermediate);
  if (w && r && w->kind == AccessPattern::OneToOne) {
    switch (r->kind) {
      case AccessPattern::OneToOne: return {Decision::Fuse, "Element-wise producer/consumer"};
      case AccessPattern::Reduction: return {Decision::Fuse, "Map-reduce pattern"};
      case AccessPattern::Stencil:
        if (r->offsets.size() <= 3) return {Decision::MaybeFuse, "Small stencil - profile to decide"};
        return {Decision::DontFuse, "Large stencil radius - keep separate"};
      case AccessPattern::Gather: return {Decision::DontFuse, "Gather pattern - keep separate"};
      default: break;
    }
  }
  return {Decision::MaybeFuse, "Unknown pattern - profile to decide"};
}

AutoFused auto_fuse_pipeline(const std::vector<Kernel> &kernels) {
  if (kernels.empty()) throw EmptyPipeline("auto_fuse_pipeline: cannot fuse empty kernel list");
  AutoFused out;
  out.kernel = kernels[0];
  for (size_t i = 1; i < kernels.size(); ++i) {
    const Kernel &k = kernels[i];
    const std::vector<std::string> writes = names_of(analyze(out.kernel).writes),
                                   reads = names_of(analyze(k).reads);
    const std::string *inter = nullptr;
    for (auto &w : writes)
      if (contains(reads, w)) {
        inter = &w;
        break;
      }
    if (!inter) {
      out.kernel = k;
      continue;
    }
    const Hint hint = should_fuse(out.kernel, k, *inter);
    std::optional<Kernel> fused;
    if (hint.decision == Decision::Fuse) fused = try_fuse(out.kernel, k, *inter);
    if (fused) {
      out.eliminated.insert(out.eliminated.begin(), *inter);
      out.kernel = *fused;
    } else {
      out.skipped.insert(out.skipped.begin(), hint.reason);
      out.kernel = k;
    }
  }
  return out;
}

std::string analyze_pipeline(const std::vector<Kernel> &kernels) {
  std::string out = "=== Fusion Analysis ===\n";
  for (size_t i = 0; i + 1 < kernels.size(); ++i) {
    const Kernel &prod = kernels[i], &cons = kernels[i + 1];
    const Info p = analyze(prod), c = analyze(cons);
    out += "\n[" + std::to_string(i) + "] " + prod.name + " -> " + cons.name + "\n";
    for (auto &w : p.writes) {
      if (!find(c.reads, w.first)) continue;
      const Hint hint = should_fuse(prod, cons, w.first);
      const char *symbol = hint.decision == Decision::Fuse ? "[FUSE]"
                           : hint.decision == Decision::DontFuse ? "[SKIP]" : "[MAYBE]";
      out += std::string("  ") + symbol + " via '" + w.first + "': " + hint.reason + "\n";
    }
  }
  return out + "\n";
}

std::string print_pattern(const AccessPattern &p) {
  switch (p.kind) {
    case AccessPattern::OneToOne: return "(one_to_one " + print_expr(p.index) + ")";
    case AccessPattern::Stencil: {
      std::string s = "(stencil";
      for (int o : p.offsets) s += " " + std::to_string(o);
      return s + ")";
    }
    case AccessPattern::Reduction: return std::string("(reduction ") + binop_name(p.op) + ")";
    case AccessPattern::Gather: return "gather";
    default: return "unknown";
  }
}

std::string print_info(const Info &info) {
  std::string s = "(info (reads";
  for (auto &r : info.reads) s += " (" + r.first + " " + print_pattern(r.second) + ")";
  s += ") (writes";
  for (auto &w : info.writes) s += " (" + w.first + " " + print_pattern(w.second) + ")";
  s += std::string(") (barriers ") + (info.has_barriers ? "true" : "false") + ") (atomics " +
       (info.has_atomics ? "true" : "false") + "))";
  return s;
}

}  // namespace fusion
}  // namespace ir
}  // namespace sarek_hip
