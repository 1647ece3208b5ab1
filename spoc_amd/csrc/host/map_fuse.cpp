// Element-wise kernels as a class: `if tid < n then out[tid] <- f(in_1[tid], ..., in_k[tid], scalars, tid)`, the shape
// of the reference's vector add, stream triad and saxpy kernels (benchmarks/bench_vector_add.ml:53-61,
// bench_stream_triad.ml:22-32) and of any map a user writes.  The generated kernel for such an IR moves one element per
// thread; what is built here from the same IR is the stream kernels' shape instead -- four 128-bit loads per input in
// flight per thread, non-temporal stores, a wave owning four consecutive KiB -- with the kernel's own expression, as
// the lowering prints it, applied to every element, and optionally the block-256 sums of the result (the reference's
// tree kernel, benchmarks/bench_reduction.ml:62-96, one wave reduction per 256 elements) in the same pass.
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <optional>
#include <string>
#include <vector>

#include "ir.hpp"
#include "map_fuse.hpp"

namespace sarek_hip {
namespace ir {
namespace {

bool is_var(const ExprP &e, const std::string &name) { return e && e->kind == Expr::VarRef && e->var.name == name; }

bool is_intr(const ExprP &e, const char *name) { return e && e->kind == Expr::Intrinsic && e->name == name; }

// threadIdx.x + blockIdx.x * blockDim.x in any of the orders a kernel text writes it
bool is_global_id(const ExprP &e) {
  if (is_intr(e, "global_thread_id") || is_intr(e, "global_idx") || is_intr(e, "global_idx_x")) return true;
  if (!e || e->kind != Expr::BinopE || e->binop != Binop::Add) return false;
  for (int t = 0; t < 2; ++t) {
    const ExprP &tx = e->args[t], &prod = e->args[1 - t];
    if (!(is_intr(tx, "thread_idx_x") || is_intr(tx, "thread_id_x"))) continue;
    if (!prod || prod->kind != Expr::BinopE || prod->binop != Binop::Mul) continue;
    for (int u = 0; u < 2; ++u) {
      const ExprP &bi = prod->args[u], &bd = prod->args[1 - u];
      if ((is_intr(bi, "block_idx_x") || is_intr(bi, "block_id_x")) && is_intr(bd, "block_dim_x")) return true;
    }
  }
  return false;
}

// Names the rebuilt texts use themselves: everything of their own carries the prefix sarek_f_ (the loop variables of
// the kernel bodies included), the element variables the suffix __e.  A parameter spelled like that would be shadowed
// there, so such a kernel stays with the generated code; any other name, however short, is the kernel's to use.
// What sarek_f_apply declares before the kernel's own statements: the inputs' element values, the scalars, the
// element's index and the result.
std::vector<std::string> element_function_names(const MapKernel &m) {
  std::vector<std::string> names{m.tid, "sarek_f_res"};
  for (const auto &p : m.params) names.push_back(p.kind == MapKernel::Param::Vec ? p.name + "__e" : p.name);
  return names;
}

bool name_is_free(const std::string &n) {
  return n.compare(0, 8, "sarek_f_") != 0 && !(n.size() > 3 && n.compare(n.size() - 3, 3, "__e") == 0);
}

struct Matcher {
  MapKernel m;
  std::vector<std::string> bound;   // immutable let variables in scope

  int param_index(const std::string &name) const {
    for (size_t i = 0; i < m.params.size(); ++i)
      if (m.params[i].name == name) return static_cast<int>(i);
    return -1;
  }

  // An expression whose value depends on nothing but the element's inputs, the scalars and tid
  bool pure(const ExprP &e) {
    if (!e) return false;
    switch (e->kind) {
      case Expr::ConstInt32: case Expr::ConstInt64: case Expr::ConstFloat32: case Expr::ConstFloat64:
      case Expr::ConstBool:
        return true;
      case Expr::VarRef: {
        if (e->var.is_mutable) return false;
        if (e->var.name == m.tid) return true;
        if (std::find(bound.begin(), bound.end(), e->var.name) != bound.end()) return true;
        const int p = param_index(e->var.name);
        return p >= 0 && m.params[p].kind != MapKernel::Param::Vec;
      }
      case Expr::BinopE: return e->args.size() == 2 && pure(e->args[0]) && pure(e->args[1]);
      case Expr::UnopE: return e->args.size() == 1 && pure(e->args[0]);
      case Expr::If: return e->args.size() == 3 && pure(e->args[0]) && pure(e->args[1]) && pure(e->args[2]);
      case Expr::Cast:
        if (!e->type || e->args.size() != 1) return false;
        if (e->type->kind != Type::Int32 && e->type->kind != Type::Int64 && e->type->kind != Type::Float32 &&
            e->type->kind != Type::Float64)
          return false;
        return pure(e->args[0]);
      case Expr::ArrayRead: {
        const int p = param_index(e->name);
        if (p < 0 || m.params[p].kind != MapKernel::Param::Vec || p == m.out) return false;
        if (e->args.size() != 1 || !is_var(e->args[0], m.tid)) return false;
        if (std::find(m.inputs.begin(), m.inputs.end(), p) == m.inputs.end()) m.inputs.push_back(p);
        return true;
      }
      case Expr::Intrinsic: {
        static const char *math[] = {"sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh", "tanh", "exp",
                                     "exp2", "log", "log2", "log10", "sqrt", "rsqrt", "cbrt", "floor", "ceil",
                                     "round", "trunc", "fabs", "atan2", "pow", "fma", "min", "max"};
        if (e->has_templ) return false;
        bool known = false;
        for (const char *n : math) known = known || e->name == n;
        if (!known) return false;
        for (const auto &a : e->args)
          if (!pure(a)) return false;
        return true;
      }
      default: return false;
    }
  }

  // reads of in[tid] become the element's variable in__e
  ExprP rewrite(const ExprP &e) {
    if (e->kind == Expr::ArrayRead) {
      auto v = std::make_shared<Expr>();
      v->kind = Expr::VarRef;
      v->var.name = e->name + "__e";
      return v;
    }
    if (e->args.empty()) return e;
    auto c = std::make_shared<Expr>(*e);
    for (auto &a : c->args) a = rewrite(a);
    return c;
  }

  // S := let x = E in S | out[tid] <- E, through single-statement blocks and sequences
  std::optional<StmtP> body(const StmtP &s) {
    if (!s) return std::nullopt;
    switch (s->kind) {
      case Stmt::Block:
      case Stmt::Seq:
        if (s->stmts.size() != 1) return std::nullopt;
        return body(s->stmts[0]);
      case Stmt::Let: {
        if (s->var.is_mutable || !s->e || s->e->kind == Expr::ArrayCreate || !pure(s->e)) return std::nullopt;
        // A let may take a scalar parameter's name (the lowering gives the new variable a name of its own); one that
        // hides the index or a vector would change what the reads and the store mean.
        const int hidden = param_index(s->var.name);
        if (s->var.name == m.tid || !name_is_free(s->var.name) ||
            (hidden >= 0 && m.params[hidden].kind == MapKernel::Param::Vec))
          return std::nullopt;
        if (s->stmts.size() != 1) return std::nullopt;
        bound.push_back(s->var.name);
        auto inner = body(s->stmts[0]);
        bound.pop_back();
        if (!inner) return std::nullopt;
        auto c = std::make_shared<Stmt>(*s);
        c->e = rewrite(s->e);
        c->stmts[0] = *inner;
        return StmtP(c);
      }
      case Stmt::Assign: {
        if (!s->lhs || s->lhs->kind != LValue::LArrayElem || param_index(s->lhs->name) != m.out) return std::nullopt;
        if (!is_var(s->lhs->index, m.tid) || !pure(s->e)) return std::nullopt;
        auto lhs = std::make_shared<LValue>();
        lhs->kind = LValue::LVar;
        lhs->var.name = "sarek_f_res";
        auto c = std::make_shared<Stmt>(*s);
        c->lhs = lhs;
        c->e = rewrite(s->e);
        return StmtP(c);
      }
      default: return std::nullopt;
    }
  }
};

// the first assignment target under the lets: names the output vector before the purity walk needs it
const Stmt *find_assign(const StmtP &s) {
  const Stmt *p = s.get();
  while (p) {
    if (p->kind == Stmt::Assign) return p;
    if ((p->kind == Stmt::Block || p->kind == Stmt::Seq || p->kind == Stmt::Let) && p->stmts.size() == 1)
      p = p->stmts[0].get();
    else
      return nullptr;
  }
  return nullptr;
}

}  // namespace

std::optional<MapKernel> match_map(const Kernel &k) {
  if (!k.funcs.empty() || !k.locals.empty() || !k.types.empty() || !k.variants.empty() || !k.body) return std::nullopt;
  Matcher mt;
  MapKernel &m = mt.m;
  for (const Decl &d : k.params) {
    if (d.kind != Decl::Param || !d.var.type) return std::nullopt;
    MapKernel::Param p;
    p.name = d.var.name;
    if (!name_is_free(p.name)) return std::nullopt;
    const Type &t = *d.var.type;
    if (t.kind == Type::Vec && t.elt && t.elt->kind == Type::Float32) p.kind = MapKernel::Param::Vec;
    else if (t.kind == Type::Float32) p.kind = MapKernel::Param::F32;
    else if (t.kind == Type::Int32) p.kind = MapKernel::Param::I32;
    else return std::nullopt;
    for (const auto &q : m.params)
      if (q.name == p.name) return std::nullopt;
    m.params.push_back(p);
  }
  // let tid = <global id> in if tid < n then S
  const Stmt *s = k.body.get();
  while ((s->kind == Stmt::Block || s->kind == Stmt::Seq) && s->stmts.size() == 1) s = s->stmts[0].get();
  if (s->kind != Stmt::Let || s->var.is_mutable || !is_global_id(s->e) || s->stmts.size() != 1) return std::nullopt;
  if (!s->var.type || s->var.type->kind != Type::Int32) return std::nullopt;
  m.tid = s->var.name;
  if (mt.param_index(m.tid) >= 0 || !name_is_free(m.tid)) return std::nullopt;
  const Stmt *guard = s->stmts[0].get();
  while ((guard->kind == Stmt::Block || guard->kind == Stmt::Seq) && guard->stmts.size() == 1)
    guard = guard->stmts[0].get();
  if (guard->kind != Stmt::If || !guard->e || guard->stmts.empty()) return std::nullopt;
  if (guard->stmts.size() > 1 && guard->stmts[1] && guard->stmts[1]->kind != Stmt::Empty) return std::nullopt;
  const Expr &c = *guard->e;
  if (c.kind != Expr::BinopE || c.binop != Binop::Lt || !is_var(c.args[0], m.tid) || !c.args[1] ||
      c.args[1]->kind != Expr::VarRef)
    return std::nullopt;
  m.n = mt.param_index(c.args[1]->var.name);
  if (m.n < 0 || m.params[m.n].kind != MapKernel::Param::I32) return std::nullopt;
  const Stmt *assign = find_assign(guard->stmts[0]);
  if (!assign || !assign->lhs || assign->lhs->kind != LValue::LArrayElem) return std::nullopt;
  m.out = mt.param_index(assign->lhs->name);
  if (m.out < 0 || m.params[m.out].kind != MapKernel::Param::Vec) return std::nullopt;
  auto rewritten = mt.body(guard->stmts[0]);
  if (!rewritten) return std::nullopt;
  std::sort(m.inputs.begin(), m.inputs.end());
  if (m.inputs.size() > 6) return std::nullopt;   // registers: four 128-bit loads per input and thread
  FunctionScope element_function(element_function_names(m));
  m.body = gen_stmt(*rewritten, "  ");
  return m;
}

namespace {

// What both rebuilt kernels start with: the vector type, the wave reduction (when sums are wanted), the element
// function sarek_f_apply(<inputs' values>, <scalars>, <index>) holding the kernel's own statements, and
// sarek_f_opaque.  `actuals_tail` receives the scalar arguments of a call ("alpha, k, ").
std::string prelude(const MapKernel &m, bool with_sums, std::string *actuals_tail) {
  std::string o;
  // no contraction of products into sums, here as in the generated text of the same kernel: the two texts then
  // round the expression's operations alike whatever code surrounds them
  o += "#pragma clang fp contract(off)\n";
  o += "typedef float sarek_f_v4 __attribute__((ext_vector_type(4)));\n";
  if (with_sums) {
    // the stream kernels' wave reduction: quad_perm, row_half_mirror, row_mirror, then the four rows
    o += "template <int Ctrl> __device__ __forceinline__ float sarek_f_dpp_add(float v) {\n"
         "  int sh = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), Ctrl, 0xF, 0xF, true);\n"
         "  return v + __builtin_bit_cast(float, sh);\n}\n"
         "__device__ __forceinline__ float sarek_f_wave_sum(float v) {\n"
         "  v = sarek_f_dpp_add<0xB1>(v);\n  v = sarek_f_dpp_add<0x4E>(v);\n  v = sarek_f_dpp_add<0x141>(v);\n"
         "  v = sarek_f_dpp_add<0x140>(v);\n  int iv = __builtin_bit_cast(int, v);\n"
         "  float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 0));\n"
         "  float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 16));\n"
         "  float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 32));\n"
         "  float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 48));\n"
         "  return (r0 + r1) + (r2 + r3);\n}\n";
  }
  // one element: the kernel's own statements on the element's inputs
  std::string formals;
  for (int p : m.inputs) formals += "float " + m.params[p].name + "__e, ";
  for (const auto &p : m.params) {
    if (p.kind == MapKernel::Param::Vec) continue;
    formals += std::string(p.kind == MapKernel::Param::F32 ? "float " : "int ") + p.name + ", ";
    *actuals_tail += p.name + ", ";
  }
  o += "__device__ __forceinline__ float sarek_f_apply(" + formals + "int " + m.tid + ") {\n  float sarek_f_res;\n" +
       m.body + "  return sarek_f_res;\n}\n";
  // The element's value passes through an empty asm before it is stored and summed: the compiler then cannot fold
  // the expression's last multiplication into the first addition of the sum (an fma there would add a product that
  // was never rounded, and the sums would no longer be those of the stored vector).
  o += "__device__ __forceinline__ float sarek_f_opaque(float v) {\n  asm(\"\" : \"+v\"(v));\n  return v;\n}\n";
  return o;
}

// sarek_f_opaque(sarek_f_apply(...)) with `value_of` ('@' = the input's number) as each input's value
std::string apply_call(const MapKernel &m, const std::string &actuals_tail, const std::string &value_of,
                       const std::string &index) {
  std::string a = "sarek_f_opaque(sarek_f_apply(";
  for (size_t i = 0; i < m.inputs.size(); ++i) {
    std::string v = value_of;
    const size_t at = v.find('@');
    v.replace(at, 1, std::to_string(i));
    a += v + ", ";
  }
  return a + actuals_tail + "(int)(" + index + ")))";
}

std::string formal_params(const MapKernel &m) {
  std::string o;
  for (size_t i = 0; i < m.params.size(); ++i) {
    const auto &p = m.params[i];
    if (p.kind == MapKernel::Param::Vec)
      o += (static_cast<int>(i) == m.out ? "float* __restrict__ " : "const float* ") + p.name + ", ";
    else
      o += std::string(p.kind == MapKernel::Param::F32 ? "float " : "int ") + p.name + ", ";
  }
  return o;
}

}  // namespace

std::string map_source(const MapKernel &m, int reduce, bool nt_loads, uint32_t pad_bits) {
  const bool with_sums = reduce == 1, with_max = reduce == 2;
  // what slots past n count as: 0 in a sum, the maximum tree's fill value (its exact bits) in a maximum
  char pad[48] = "0.f";
  if (with_max) std::snprintf(pad, sizeof(pad), "__uint_as_float(0x%08xu)", static_cast<unsigned>(pad_bits));
  std::string actuals_tail;
  std::string o = prelude(m, with_sums, &actuals_tail);
  if (with_max) o += "__device__ __forceinline__ float sarek_f_greater(float a, float b) { return b > a ? b : a; }\n";
  auto apply = [&](const std::string &value_of, const std::string &index) {
    return apply_call(m, actuals_tail, value_of, index);
  };
  const std::string out = m.params[m.out].name;
  // eight waves per SIMD (64 registers) is the triad's measured best and fits four loads of up to two inputs; with
  // more inputs the loads alone need more registers than that, and the occupancy is left to the compiler
  o += std::string("extern \"C\" __global__ __launch_bounds__(256) ") +
       (m.inputs.size() <= 2 ? "__attribute__((amdgpu_waves_per_eu(8, 8))) " : "") + "void sarek_map(";
  o += formal_params(m) + "float* __restrict__ sarek_f_partials) {\n";
  o += "  const long long sarek_f_n = " + m.params[m.n].name + ", sarek_f_n4 = sarek_f_n >> 2;\n";
  // a wave owns four consecutive KiB of every vector: slot u of lane l is float4 number base + 64 u; the tail's share
  // of a block sum starts at -0, whose addition changes nothing (a block of elements that are all -0 sums to -0)
  o += "  const long long sarek_f_base = (long long)blockIdx.x * 1024 + (threadIdx.x >> 6) * 256 + (threadIdx.x & 63);\n"
       "  const bool sarek_f_full = sarek_f_base + 192 < sarek_f_n4;\n"
       "  sarek_f_v4 sarek_f_r[4];\n  float sarek_f_extra[4] = {-0.f, -0.f, -0.f, -0.f};\n";
  for (size_t i = 0; i < m.inputs.size(); ++i)
    o += "  const sarek_f_v4* sarek_f_p" + std::to_string(i) + " = reinterpret_cast<const sarek_f_v4*>(" +
         m.params[m.inputs[i]].name + ");\n";
  o += "  sarek_f_v4* sarek_f_po = reinterpret_cast<sarek_f_v4*>(" + out + ");\n";
  o += "  if (sarek_f_full) {\n";
  for (size_t i = 0; i < m.inputs.size(); ++i) {
    const std::string is = std::to_string(i);
    o += "    sarek_f_v4 sarek_f_x" + is + "[4];\n#pragma unroll\n    for (int sarek_f_u = 0; sarek_f_u < 4; ++sarek_f_u) sarek_f_x" + is + "[sarek_f_u] = " +
         (nt_loads ? "__builtin_nontemporal_load(sarek_f_p" + is + " + sarek_f_base + 64 * sarek_f_u)"
                   : "sarek_f_p" + is + "[sarek_f_base + 64 * sarek_f_u]") +
         ";\n";
  }
  o += "#pragma unroll\n    for (int sarek_f_u = 0; sarek_f_u < 4; ++sarek_f_u)\n#pragma unroll\n      for (int sarek_f_j = 0; sarek_f_j < 4; ++sarek_f_j)\n"
       "        sarek_f_r[sarek_f_u][sarek_f_j] = " + apply("sarek_f_x@[sarek_f_u][sarek_f_j]", "(sarek_f_base + 64 * sarek_f_u) * 4 + sarek_f_j") + ";\n";
  o += "#pragma unroll\n    for (int sarek_f_u = 0; sarek_f_u < 4; ++sarek_f_u) __builtin_nontemporal_store(sarek_f_r[sarek_f_u], sarek_f_po + sarek_f_base + 64 * sarek_f_u);\n";
  o += "  } else {\n#pragma unroll\n    for (int sarek_f_u = 0; sarek_f_u < 4; ++sarek_f_u) {\n      const long long sarek_f_i = sarek_f_base + 64 * sarek_f_u;\n"
       "      sarek_f_r[sarek_f_u] = sarek_f_v4{0.f, 0.f, 0.f, 0.f};\n      if (sarek_f_i < sarek_f_n4) {\n";
  for (size_t i = 0; i < m.inputs.size(); ++i)
    o += "        const sarek_f_v4 sarek_f_y" + std::to_string(i) + " = sarek_f_p" + std::to_string(i) + "[sarek_f_i];\n";
  o += "#pragma unroll\n        for (int sarek_f_j = 0; sarek_f_j < 4; ++sarek_f_j) sarek_f_r[sarek_f_u][sarek_f_j] = " + apply("sarek_f_y@[sarek_f_j]", "sarek_f_i * 4 + sarek_f_j") + ";\n"
       "        sarek_f_po[sarek_f_i] = sarek_f_r[sarek_f_u];\n      }";
  {
    std::string a = "sarek_f_opaque(sarek_f_apply(";
    for (int p : m.inputs) a += m.params[p].name + "[sarek_f_k], ";
    a += actuals_tail + "(int)sarek_f_k))";
    if (with_max) {
      // the slot that holds the end of the vector takes its one to three elements; everything past n is the fill value
      o += " else {\n#pragma unroll\n        for (int sarek_f_e = 0; sarek_f_e < 4; ++sarek_f_e) {\n          const long long sarek_f_k = (sarek_f_i << 2) + sarek_f_e;\n"
           "          sarek_f_r[sarek_f_u][sarek_f_e] = " + std::string(pad) + ";\n          if (sarek_f_k < sarek_f_n) {\n            sarek_f_r[sarek_f_u][sarek_f_e] = " + a +
           ";\n            " + out + "[sarek_f_k] = sarek_f_r[sarek_f_u][sarek_f_e];\n          }\n        }\n      }\n";
    } else {
      // the lane whose slot holds the end of the vector takes the one to three elements there, summed apart (kept
      // out of the vector registers: folding them into r measured 2.7 % slower on the whole kernel)
      o += "\n      if (sarek_f_i == sarek_f_n4) {\n        for (long long sarek_f_k = sarek_f_n4 << 2; sarek_f_k < sarek_f_n; ++sarek_f_k) {\n"
           "          const float sarek_f_v = " + a + ";\n          " + out + "[sarek_f_k] = sarek_f_v;\n          sarek_f_extra[sarek_f_u] += sarek_f_v;\n        }\n      }\n";
    }
  }
  o += "    }\n  }\n";
  if (with_sums) {
    o += "  const long long sarek_f_nblocks = (sarek_f_n + 255) >> 8;\n  float sarek_f_t[4];\n#pragma unroll\n"
         "  for (int sarek_f_u = 0; sarek_f_u < 4; ++sarek_f_u)\n    sarek_f_t[sarek_f_u] = sarek_f_wave_sum(((sarek_f_r[sarek_f_u][0] + sarek_f_r[sarek_f_u][1]) + "
         "(sarek_f_r[sarek_f_u][2] + sarek_f_r[sarek_f_u][3])) + sarek_f_extra[sarek_f_u]);\n"
         "  const long long sarek_f_j0 = (long long)blockIdx.x * 16 + (threadIdx.x >> 6) * 4;\n"
         "  if ((threadIdx.x & 63) == 0) {\n    if (sarek_f_j0 + 4 <= sarek_f_nblocks) {\n"
         "      *reinterpret_cast<sarek_f_v4*>(sarek_f_partials + sarek_f_j0) = "
         "sarek_f_v4{sarek_f_t[0], sarek_f_t[1], sarek_f_t[2], sarek_f_t[3]};\n    } else {\n#pragma unroll\n"
         "      for (int sarek_f_u = 0; sarek_f_u < 4; ++sarek_f_u)\n        if (sarek_f_j0 + sarek_f_u < sarek_f_nblocks) sarek_f_partials[sarek_f_j0 + sarek_f_u] = sarek_f_t[sarek_f_u];\n"
         "    }\n  }\n";
  }
  if (with_max) {
    // the tree's comparisons in the tree's order: halves 128 .. 4 pair lane l with lanes l + 32 .. l + 1 component by
    // component, halves 2 and 1 the four components of lane 0
    o += "  const long long sarek_f_nblocks = (sarek_f_n + 255) >> 8;\n  float sarek_f_t[4];\n#pragma unroll\n"
         "  for (int sarek_f_u = 0; sarek_f_u < 4; ++sarek_f_u) {\n    sarek_f_v4 sarek_f_w = sarek_f_r[sarek_f_u];\n#pragma unroll\n"
         "    for (int sarek_f_h = 32; sarek_f_h >= 1; sarek_f_h >>= 1)\n#pragma unroll\n      for (int sarek_f_c = 0; sarek_f_c < 4; ++sarek_f_c) "
         "sarek_f_w[sarek_f_c] = sarek_f_greater(sarek_f_w[sarek_f_c], __shfl_down(sarek_f_w[sarek_f_c], sarek_f_h, 64));\n"
         "    sarek_f_t[sarek_f_u] = sarek_f_greater(sarek_f_greater(sarek_f_w[0], sarek_f_w[2]), sarek_f_greater(sarek_f_w[1], sarek_f_w[3]));\n  }\n"
         "  const long long sarek_f_j0 = (long long)blockIdx.x * 16 + (threadIdx.x >> 6) * 4;\n"
         "  if ((threadIdx.x & 63) == 0) {\n    if (sarek_f_j0 + 4 <= sarek_f_nblocks && "
         "(reinterpret_cast<unsigned long long>(sarek_f_partials) & 15ull) == 0) {\n"
         "      *reinterpret_cast<sarek_f_v4*>(sarek_f_partials + sarek_f_j0) = "
         "sarek_f_v4{sarek_f_t[0], sarek_f_t[1], sarek_f_t[2], sarek_f_t[3]};\n    } else {\n#pragma unroll\n"
         "      for (int sarek_f_u = 0; sarek_f_u < 4; ++sarek_f_u)\n        if (sarek_f_j0 + sarek_f_u < sarek_f_nblocks) sarek_f_partials[sarek_f_j0 + sarek_f_u] = sarek_f_t[sarek_f_u];\n"
         "    }\n  }\n";
  }
  o += "}\n";
  return o;
}

// The block-256 tree sum with an element-wise expression in front of it: benchmarks/bench_reduction.ml:62-96 and
// bench_dot_product.ml:16-54 with any pure f(in_1[gid], ..., scalars, gid) where they have in[gid] and a[gid] * b[gid].
// The kernel is taken apart (shared array, tid, gid, the guarded first store and its expression), put together again
// from the tree's text with that expression in its place, and accepted when the two normalise to the same form: so
// everything but the expression is the tree, to the letter.
namespace {
std::optional<MapKernel> match_tree(const Kernel &k, bool is_max) {
  if (!k.funcs.empty() || !k.locals.empty() || !k.types.empty() || !k.variants.empty() || !k.body) return std::nullopt;
  Matcher mt;
  MapKernel &m = mt.m;
  for (const Decl &d : k.params) {
    if (d.kind != Decl::Param || !d.var.type) return std::nullopt;
    MapKernel::Param p;
    p.name = d.var.name;
    if (!name_is_free(p.name)) return std::nullopt;
    const Type &t = *d.var.type;
    if (t.kind == Type::Vec && t.elt && t.elt->kind == Type::Float32) p.kind = MapKernel::Param::Vec;
    else if (t.kind == Type::Float32) p.kind = MapKernel::Param::F32;
    else if (t.kind == Type::Int32) p.kind = MapKernel::Param::I32;
    else return std::nullopt;
    for (const auto &q : m.params)
      if (q.name == p.name) return std::nullopt;
    m.params.push_back(p);
  }
  auto unwrap = [](const Stmt *s) {
    while (s && (s->kind == Stmt::Block || s->kind == Stmt::Seq) && s->stmts.size() == 1) s = s->stmts[0].get();
    return s;
  };
  // let sdata = shared f32[256] in let tid = .. in let gid = .. in seq (block (if gid < n then sdata[tid] <- LEAF else ..)) ..
  const Stmt *l0 = unwrap(k.body.get());
  if (!l0 || l0->kind != Stmt::Let || !l0->e || l0->e->kind != Expr::ArrayCreate || l0->stmts.size() != 1) return std::nullopt;
  const Stmt *l1 = unwrap(l0->stmts[0].get());
  if (!l1 || l1->kind != Stmt::Let || l1->stmts.size() != 1) return std::nullopt;
  const Stmt *l2 = unwrap(l1->stmts[0].get());
  if (!l2 || l2->kind != Stmt::Let || l2->stmts.size() != 1 || !is_global_id(l2->e)) return std::nullopt;
  const Stmt *sq = l2->stmts[0].get();
  while (sq && sq->kind == Stmt::Block && sq->stmts.size() == 1) sq = sq->stmts[0].get();
  if (!sq || sq->kind != Stmt::Seq || sq->stmts.size() < 2) return std::nullopt;
  const Stmt *first = unwrap(sq->stmts[0].get());
  if (!first || first->kind != Stmt::If || first->stmts.size() != 2 || !first->e) return std::nullopt;
  const Expr &c = *first->e;
  if (c.kind != Expr::BinopE || c.binop != Binop::Lt || !is_var(c.args[0], l2->var.name) || !c.args[1] ||
      c.args[1]->kind != Expr::VarRef)
    return std::nullopt;
  const Stmt *store = unwrap(first->stmts[0].get());
  if (!store || store->kind != Stmt::Assign || !store->lhs || store->lhs->kind != LValue::LArrayElem ||
      store->lhs->name != l0->var.name || !store->e)
    return std::nullopt;
  const Stmt *fill = unwrap(first->stmts[1].get());
  if (!fill || fill->kind != Stmt::Assign || !fill->e || fill->e->kind != Expr::ConstFloat32) return std::nullopt;
  m.is_max = is_max;
  m.pad = gen_expr(fill->e);
  m.tid = l2->var.name;
  m.n = mt.param_index(c.args[1]->var.name);
  if (m.n < 0 || m.params[m.n].kind != MapKernel::Param::I32) return std::nullopt;
  if (mt.param_index(m.tid) >= 0 || !name_is_free(m.tid)) return std::nullopt;
  // the expression first (it names the inputs), then the output: the one vector it does not read
  m.out = -1;
  if (!mt.pure(store->e)) return std::nullopt;
  for (size_t i = 0; i < m.params.size(); ++i) {
    if (m.params[i].kind != MapKernel::Param::Vec) continue;
    if (std::find(m.inputs.begin(), m.inputs.end(), static_cast<int>(i)) != m.inputs.end()) continue;
    if (m.out >= 0) return std::nullopt;   // a vector that is neither read nor the output
    m.out = static_cast<int>(i);
  }
  if (m.out < 0 || m.inputs.empty() || m.inputs.size() > 3) return std::nullopt;
  std::sort(m.inputs.begin(), m.inputs.end());
  // the tree round this expression, from the text of the reference's kernel with this kernel's names
  auto v = [](const Var &x, const char *type) { return "(var " + x.name + " " + std::to_string(x.id) + " " + type + ")"; };
  const std::string sdata = l0->var.name, tid = v(l1->var, "i32"), gid = v(l2->var, "i32");
  const std::string n = "(var " + m.params[m.n].name + " " + std::to_string(c.args[1]->var.id) + " i32)";
  const std::string slot = "(lelem " + sdata + " " + tid + ")";
  std::string steps = "(block (if (lt " + gid + " " + n + ") (assign " + slot + " " + print_expr(store->e) + ") (assign " +
                      slot + " " + (is_max ? print_expr(fill->e) : std::string("(f32 0.0)")) + "))) (barrier) ";
  for (int half = 128; half >= 1; half >>= 1) {
    const std::string h = "(i32 " + std::to_string(half) + ")";
    if (is_max) {
      // benchmarks/bench_reduction_max.ml:18-100: let a = sdata[tid], b = sdata[tid + half] in if b > a then sdata[tid] <- b
      const std::string a = "(var sarek_f_a " + std::to_string(900000 + half) + " f32)";
      const std::string b = "(var sarek_f_b " + std::to_string(910000 + half) + " f32)";
      steps += "(block (if (lt " + tid + " " + h + ") (let " + a + " (read " + sdata + " " + tid + ") (let " + b + " (read " +
               sdata + " (add " + tid + " " + h + ")) (if (gt " + b + " " + a + ") (assign " + slot + " " + b +
               ")))))) (barrier) ";
    } else {
      steps += "(block (if (lt " + tid + " " + h + ") (assign " + slot + " (add (read " + sdata + " " + tid + ") (read " +
               sdata + " (add " + tid + " " + h + ")))))) (barrier) ";
    }
  }
  steps += "(block (if (eq " + tid + " (i32 0)) (assign (lelem " + m.params[m.out].name +
           " (intr (Gpu) block_idx_x)) (read " + sdata + " (i32 0)))))";
  const std::string want = canonical_form(k);
  bool same = false;
  for (int trailing = 0; trailing < 2 && !same; ++trailing) {
    const std::string body = "(let " + v(l0->var, "(array f32 shared)") + " (newarray f32 (i32 256) shared) (let " + tid +
                             " (intr (Gpu) thread_idx_x) (let " + gid +
                             " (add (intr (Gpu) thread_idx_x) (mul (intr (Gpu) block_dim_x) (intr (Gpu) block_idx_x))) (seq " +
                             steps + (trailing ? " (barrier)" : "") + "))))";
    Kernel again = k;
    try {
      again.body = parse_stmt(body);
      same = canonical_form(again) == want;
    } catch (const std::exception &) {
      return std::nullopt;
    }
  }
  if (!same) return std::nullopt;
  auto lhs = std::make_shared<LValue>();
  lhs->kind = LValue::LVar;
  lhs->var.name = "sarek_f_res";
  auto st = std::make_shared<Stmt>();
  st->kind = Stmt::Assign;
  st->lhs = lhs;
  st->e = mt.rewrite(store->e);
  FunctionScope element_function(element_function_names(m));
  m.body = gen_stmt(StmtP(st), "  ");
  return m;
}
}  // namespace

std::optional<MapKernel> match_tree_sum(const Kernel &k) { return match_tree(k, false); }
std::optional<MapKernel> match_tree_max(const Kernel &k) { return match_tree(k, true); }

// One input: lane l of a wave holds elements l, l + 64, l + 128, l + 192 of a block (the hand maximum's layout: two
// comparisons inside the lane, then six across lanes per block; with 128-bit loads the same tree needs 24 cross-lane
// steps per block, and a 4-byte-per-element kernel is bound by them: 260 against 163 us at n = 2^28).
namespace {
std::string tree_max_source_scalar_loads(const MapKernel &m) {
  std::string actuals_tail;
  std::string o = prelude(m, false, &actuals_tail);
  const std::string out = m.params[m.out].name;
  o += "__device__ __forceinline__ float sarek_f_greater(float a, float b) { return b > a ? b : a; }\n";
  o += "extern \"C\" __global__ __launch_bounds__(256) void sarek_tree(" + formal_params(m);
  o.resize(o.size() - 2);
  // (comparisons do not contract with anything: the element's value needs no asm in front of them)
  std::string a = "sarek_f_apply(";
  for (int p : m.inputs) a += "__builtin_nontemporal_load(" + m.params[p].name + " + sarek_f_i), ";
  a += actuals_tail + "(int)sarek_f_i)";
  o += ") {\n  const long long sarek_f_n = " + m.params[m.n].name + ", sarek_f_nblocks = (sarek_f_n + 255) >> 8;\n"
       "  const int sarek_f_lane = threadIdx.x & 63;\n"
       "  const long long sarek_f_j0 = ((long long)blockIdx.x * 4 + (threadIdx.x >> 6)) * 8;\n"
       "  if (sarek_f_j0 >= sarek_f_nblocks) return;\n"
       "  const bool sarek_f_full = (sarek_f_j0 + 8) * 256 <= sarek_f_n;\n  float sarek_f_m[8];\n"
       // all 32 loads of a thread are asked for before the first comparison
       "  float sarek_f_w[8][4];\n  if (sarek_f_full) {\n#pragma unroll\n    for (int sarek_f_u = 0; sarek_f_u < 8; ++sarek_f_u)\n#pragma unroll\n      for (int sarek_f_q = 0; sarek_f_q < 4; ++sarek_f_q) {\n"
       "        const long long sarek_f_i = (sarek_f_j0 + sarek_f_u) * 256 + sarek_f_lane + 64 * sarek_f_q;\n"
       "        sarek_f_w[sarek_f_u][sarek_f_q] = " + a + ";\n      }\n  } else {\n"
       "#pragma unroll\n    for (int sarek_f_u = 0; sarek_f_u < 8; ++sarek_f_u)\n#pragma unroll\n      for (int sarek_f_q = 0; sarek_f_q < 4; ++sarek_f_q) {\n"
       "        const long long sarek_f_i = (sarek_f_j0 + sarek_f_u) * 256 + sarek_f_lane + 64 * sarek_f_q;\n"
       "        sarek_f_w[sarek_f_u][sarek_f_q] = " + m.pad + ";\n        if (sarek_f_i < sarek_f_n) sarek_f_w[sarek_f_u][sarek_f_q] = " + a + ";\n      }\n  }\n"
       "#pragma unroll\n  for (int sarek_f_u = 0; sarek_f_u < 8; ++sarek_f_u) {\n    const float* sarek_f_v = sarek_f_w[sarek_f_u];\n"
       "    float sarek_f_g = sarek_f_greater(sarek_f_greater(sarek_f_v[0], sarek_f_v[2]), sarek_f_greater(sarek_f_v[1], sarek_f_v[3]));\n"
       "#pragma unroll\n    for (int sarek_f_h = 32; sarek_f_h >= 1; sarek_f_h >>= 1) sarek_f_g = sarek_f_greater(sarek_f_g, __shfl_down(sarek_f_g, sarek_f_h, 64));\n"
       "    sarek_f_m[sarek_f_u] = sarek_f_g;\n  }\n  if (sarek_f_lane != 0) return;\n"
       "  if (sarek_f_j0 + 8 <= sarek_f_nblocks && (reinterpret_cast<unsigned long long>(" + out + ") & 15ull) == 0) {\n"
       "    sarek_f_v4* sarek_f_o4 = reinterpret_cast<sarek_f_v4*>(" + out + " + sarek_f_j0);\n"
       "    sarek_f_o4[0] = sarek_f_v4{sarek_f_m[0], sarek_f_m[1], sarek_f_m[2], sarek_f_m[3]};\n"
       "    sarek_f_o4[1] = sarek_f_v4{sarek_f_m[4], sarek_f_m[5], sarek_f_m[6], sarek_f_m[7]};\n  } else {\n"
       "#pragma unroll\n    for (int sarek_f_u = 0; sarek_f_u < 8; ++sarek_f_u)\n      if (sarek_f_j0 + sarek_f_u < sarek_f_nblocks) " + out + "[sarek_f_j0 + sarek_f_u] = sarek_f_m[sarek_f_u];\n  }\n}\n";
  return o;
}

}  // namespace

// The maximum tree in the block-256 sum's load shape: lane l of a wave holds elements 4l .. 4l+3 of a block (128-bit
// loads, eight blocks per wave, all asked for before the first comparison), and the comparisons are the tree's in
// the tree's order with its strict ">" (halves 128 .. 4 across lanes component by component, 2 and 1 inside lane 0),
// so NaNs and signed zeros come out as from the tree; slots past n hold the kernel's fill value.  Two or three inputs:
// the loads are what counts there (339 against 359 us for max |x - y| at n = 2^28).
std::string tree_max_source(const MapKernel &m) {
  if (m.inputs.size() == 1) return tree_max_source_scalar_loads(m);
  std::string actuals_tail;
  std::string o = prelude(m, false, &actuals_tail);
  const std::string out = m.params[m.out].name;
  // (comparisons do not contract with anything: the element's value needs no asm in front of them)
  auto apply = [&](const std::string &value_of, const std::string &index) {
    std::string a = "sarek_f_apply(";
    for (size_t i = 0; i < m.inputs.size(); ++i) {
      std::string v = value_of;
      v.replace(v.find('@'), 1, std::to_string(i));
      a += v + ", ";
    }
    return a + actuals_tail + "(int)(" + index + "))";
  };
  o += "__device__ __forceinline__ float sarek_f_greater(float a, float b) { return b > a ? b : a; }\n"
       // lane l holds elements 4l .. 4l+3 of a block: halves 128 .. 4 pair lane l with lanes l + 32 .. l + 1 component
       // by component, halves 2 and 1 the four components of lane 0
       "__device__ __forceinline__ float sarek_f_tree_max(sarek_f_v4 w) {\n#pragma unroll\n"
       "  for (int h = 32; h >= 1; h >>= 1)\n#pragma unroll\n    for (int c = 0; c < 4; ++c) "
       "w[c] = sarek_f_greater(w[c], __shfl_down(w[c], h, 64));\n"
       "  return sarek_f_greater(sarek_f_greater(w[0], w[2]), sarek_f_greater(w[1], w[3]));\n}\n";
  o += "extern \"C\" __global__ __launch_bounds__(256) void sarek_tree(" + formal_params(m);
  o.resize(o.size() - 2);
  o += ") {\n  const long long sarek_f_n = " + m.params[m.n].name + ", sarek_f_nblocks = (sarek_f_n + 255) >> 8;\n"
       "  const int sarek_f_lane = threadIdx.x & 63;\n"
       "  const long long sarek_f_j0 = ((long long)blockIdx.x * 4 + (threadIdx.x >> 6)) * 8;\n"
       "  if (sarek_f_j0 >= sarek_f_nblocks) return;\n  float sarek_f_m[8];\n"
       "  if ((sarek_f_j0 + 8) * 256 <= sarek_f_n) {\n";
  for (size_t i = 0; i < m.inputs.size(); ++i) {
    const std::string is = std::to_string(i), name = m.params[m.inputs[i]].name;
    o += "    sarek_f_v4 sarek_f_x" + is + "[8];\n#pragma unroll\n    for (int sarek_f_u = 0; sarek_f_u < 8; ++sarek_f_u) sarek_f_x" + is +
         "[sarek_f_u] = __builtin_nontemporal_load(reinterpret_cast<const sarek_f_v4*>(" + name +
         " + (sarek_f_j0 + sarek_f_u) * 256) + sarek_f_lane);\n";
  }
  o += "#pragma unroll\n    for (int sarek_f_u = 0; sarek_f_u < 8; ++sarek_f_u) {\n      sarek_f_v4 sarek_f_w;\n#pragma unroll\n"
       "      for (int sarek_f_j = 0; sarek_f_j < 4; ++sarek_f_j) sarek_f_w[sarek_f_j] = " +
       apply("sarek_f_x@[sarek_f_u][sarek_f_j]", "(sarek_f_j0 + sarek_f_u) * 256 + sarek_f_lane * 4 + sarek_f_j") +
       ";\n      sarek_f_m[sarek_f_u] = sarek_f_tree_max(sarek_f_w);\n    }\n  } else {\n";
  {
    // the group that holds the end of the input: slots past n hold the kernel's fill value
    std::string a = "sarek_f_apply(";
    for (int p : m.inputs) a += m.params[p].name + "[sarek_f_k], ";
    a += actuals_tail + "(int)sarek_f_k)";
    o += "#pragma unroll\n    for (int sarek_f_u = 0; sarek_f_u < 8; ++sarek_f_u) {\n      sarek_f_v4 sarek_f_w;\n#pragma unroll\n"
         "      for (int sarek_f_j = 0; sarek_f_j < 4; ++sarek_f_j) {\n        const long long sarek_f_k = (sarek_f_j0 + sarek_f_u) * 256 + sarek_f_lane * 4 + sarek_f_j;\n"
         "        sarek_f_w[sarek_f_j] = " + m.pad + ";\n        if (sarek_f_k < sarek_f_n) sarek_f_w[sarek_f_j] = " + a + ";\n      }\n"
         "      sarek_f_m[sarek_f_u] = sarek_f_tree_max(sarek_f_w);\n    }\n  }\n";
  }
  o += "  if (sarek_f_lane != 0) return;\n"
       "  if (sarek_f_j0 + 8 <= sarek_f_nblocks && (reinterpret_cast<unsigned long long>(" + out + ") & 15ull) == 0) {\n"
       "    sarek_f_v4* sarek_f_o4 = reinterpret_cast<sarek_f_v4*>(" + out + " + sarek_f_j0);\n"
       "    sarek_f_o4[0] = sarek_f_v4{sarek_f_m[0], sarek_f_m[1], sarek_f_m[2], sarek_f_m[3]};\n"
       "    sarek_f_o4[1] = sarek_f_v4{sarek_f_m[4], sarek_f_m[5], sarek_f_m[6], sarek_f_m[7]};\n  } else {\n"
       "#pragma unroll\n    for (int sarek_f_u = 0; sarek_f_u < 8; ++sarek_f_u)\n      if (sarek_f_j0 + sarek_f_u < sarek_f_nblocks) " + out + "[sarek_f_j0 + sarek_f_u] = sarek_f_m[sarek_f_u];\n  }\n}\n";
  return o;
}

// The hand block-256 kernel's shape (a wave takes eight consecutive 256-element blocks, all loads issued before
// the first use, one DPP wave reduction per block, the eight sums stored as two 16-byte pieces) with the kernel's
// expression on every element: `sarek_tree(<the kernel's parameters>)`, 256 threads, ceil(ceil(n / 256) / 32) workgroups.
std::string tree_sum_source(const MapKernel &m, bool nt_loads) {
  std::string actuals_tail;
  std::string o = prelude(m, true, &actuals_tail);
  const std::string out = m.params[m.out].name;
  o += "extern \"C\" __global__ __launch_bounds__(256) void sarek_tree(" + formal_params(m);
  o.resize(o.size() - 2);   // the ", " after the last parameter
  o += ") {\n  const long long sarek_f_n = " + m.params[m.n].name + ", sarek_f_nblocks = (sarek_f_n + 255) >> 8;\n"
       "  const int sarek_f_lane = threadIdx.x & 63;\n"
       "  const long long sarek_f_j0 = ((long long)blockIdx.x * 4 + (threadIdx.x >> 6)) * 8;\n"
       "  if (sarek_f_j0 >= sarek_f_nblocks) return;\n  float sarek_f_r[8];\n"
       "  if ((sarek_f_j0 + 8) * 256 <= sarek_f_n) {\n";
  for (size_t i = 0; i < m.inputs.size(); ++i) {
    const std::string is = std::to_string(i), name = m.params[m.inputs[i]].name;
    const std::string at = "reinterpret_cast<const sarek_f_v4*>(" + name + " + (sarek_f_j0 + sarek_f_u) * 256) + sarek_f_lane";
    o += "    sarek_f_v4 sarek_f_x" + is + "[8];\n#pragma unroll\n    for (int sarek_f_u = 0; sarek_f_u < 8; ++sarek_f_u) sarek_f_x" + is + "[sarek_f_u] = " +
         (nt_loads ? "__builtin_nontemporal_load(" + at + ")" : "*(" + at + ")") + ";\n";
  }
  o += "#pragma unroll\n    for (int sarek_f_u = 0; sarek_f_u < 8; ++sarek_f_u) {\n      float sarek_f_v[4];\n#pragma unroll\n      for (int sarek_f_j = 0; sarek_f_j < 4; ++sarek_f_j) sarek_f_v[sarek_f_j] = " +
       apply_call(m, actuals_tail, "sarek_f_x@[sarek_f_u][sarek_f_j]", "(sarek_f_j0 + sarek_f_u) * 256 + sarek_f_lane * 4 + sarek_f_j") +
       ";\n      sarek_f_r[sarek_f_u] = sarek_f_wave_sum((sarek_f_v[0] + sarek_f_v[1]) + (sarek_f_v[2] + sarek_f_v[3]));\n    }\n"
       "    if (sarek_f_lane == 0) {\n      if ((reinterpret_cast<unsigned long long>(" + out + ") & 15ull) == 0) {\n"
       "        sarek_f_v4* sarek_f_o4 = reinterpret_cast<sarek_f_v4*>(" + out + " + sarek_f_j0);\n"
       "        sarek_f_o4[0] = sarek_f_v4{sarek_f_r[0], sarek_f_r[1], sarek_f_r[2], sarek_f_r[3]};\n"
       "        sarek_f_o4[1] = sarek_f_v4{sarek_f_r[4], sarek_f_r[5], sarek_f_r[6], sarek_f_r[7]};\n      } else {\n"
       "#pragma unroll\n        for (int sarek_f_u = 0; sarek_f_u < 8; ++sarek_f_u) " + out + "[sarek_f_j0 + sarek_f_u] = sarek_f_r[sarek_f_u];\n      }\n    }\n"
       "    return;\n  }\n";
  // the group that holds the end of the input
  {
    std::string a = "sarek_f_opaque(sarek_f_apply(";
    for (int p : m.inputs) a += m.params[p].name + "[sarek_f_i + sarek_f_e], ";
    a += actuals_tail + "(int)(sarek_f_i + sarek_f_e)))";
    o += "  for (int sarek_f_u = 0; sarek_f_u < 8 && sarek_f_j0 + sarek_f_u < sarek_f_nblocks; ++sarek_f_u) {\n"
         "    const long long sarek_f_i = (sarek_f_j0 + sarek_f_u) * 256 + sarek_f_lane * 4;\n    float sarek_f_t[4];\n"
         "    for (int sarek_f_e = 0; sarek_f_e < 4; ++sarek_f_e) sarek_f_t[sarek_f_e] = sarek_f_i + sarek_f_e < sarek_f_n ? " + a + " : 0.f;\n"
         "    float sarek_f_v = sarek_f_wave_sum((sarek_f_t[0] + sarek_f_t[1]) + (sarek_f_t[2] + sarek_f_t[3]));\n"
         "    if (sarek_f_lane == 0) " + out + "[sarek_f_j0 + sarek_f_u] = sarek_f_v;\n  }\n}\n";
  }
  return o;
}

}  // namespace ir
}  // namespace sarek_hip
