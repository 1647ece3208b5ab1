// C ABI of the IR fusion pass (sarek/sarek/Sarek_fusion.ml): IR text in, IR text out.
#include <cstring>
#include <string>
#include <vector>

#include "common.hpp"
#include "host/fusion.hpp"

using namespace sarek_hip;
namespace fu = sarek_hip::ir::fusion;

namespace {

int deliver(const std::string &text, char *out, size_t out_len, size_t *needed, const char *what) {
  if (needed) *needed = text.size() + 1;
  if (!out || out_len < text.size() + 1)
    return fail(SAREK_HIP_E_BUFFER_TOO_SMALL, "%s: output needs %zu bytes", what, text.size() + 1);
  std::memcpy(out, text.c_str(), text.size() + 1);
  return SAREK_HIP_OK;
}

// Runs `body`, mapping the reader's and the pass's exceptions to status codes.
template <class F>
int guarded(const char *what, F body) {
  try {
    return body();
  } catch (const ir::ParseError &e) {
    return fail(SAREK_HIP_E_PARSE, "%s: %s", what, e.what());
  } catch (const fu::EmptyPipeline &e) {
    return fail(SAREK_HIP_E_INVALID_ARG, "%s", e.what());
  } catch (const std::exception &e) {
    return fail(SAREK_HIP_E_CODEGEN, "%s: %s", what, e.what());
  }
}

bool read_kernels(const char *const *texts, int n, std::vector<ir::Kernel> &out) {
  if (n < 0 || (n > 0 && !texts)) return false;
  for (int i = 0; i < n; ++i) {
    if (!texts[i]) return false;
    out.push_back(ir::parse_kernel(texts[i]));
  }
  return true;
}

}  // namespace

extern "C" {

int sarek_hip_fusion_analyze(const char *kernel_ir, char *out, size_t out_len, size_t *needed) {
  if (!kernel_ir) return fail(SAREK_HIP_E_INVALID_ARG, "fusion_analyze: NULL IR text");
  return guarded("fusion_analyze", [&] {
    return deliver(fu::print_info(fu::analyze(ir::parse_kernel(kernel_ir))), out, out_len, needed,
                   "fusion_analyze");
  });
}

int sarek_hip_fusion_can_fuse(const char *producer_ir, const char *consumer_ir, const char *intermediate,
                              int mode, int *result) {
  if (!producer_ir || !consumer_ir || !intermediate || !result)
    return fail(SAREK_HIP_E_INVALID_ARG, "fusion_can_fuse: NULL argument");
  return guarded("fusion_can_fuse", [&] {
    const ir::Kernel p = ir::parse_kernel(producer_ir), c = ir::parse_kernel(consumer_ir);
    switch (mode) {
      case SAREK_HIP_FUSION_VERTICAL: *result = fu::can_fuse(p, c, intermediate); break;
      case SAREK_HIP_FUSION_REDUCTION: *result = fu::can_fuse_reduction(p, c, intermediate); break;
      case SAREK_HIP_FUSION_STENCIL: *result = fu::can_fuse_stencil(p, c, intermediate); break;
      case SAREK_HIP_FUSION_TRY: *result = fu::try_fuse(p, c, intermediate).has_value(); break;
      case SAREK_HIP_FUSION_TRY_ALL: *result = fu::try_fuse_all(p, c, intermediate).has_value(); break;
      default: return fail(SAREK_HIP_E_INVALID_ARG, "fusion_can_fuse: unknown mode %d", mode);
    }
    return static_cast<int>(SAREK_HIP_OK);
  });
}

int sarek_hip_fusion_fuse(const char *producer_ir, const char *consumer_ir, const char *intermediate, int mode,
                          int *fused, char *out, size_t out_len, size_t *needed) {
  if (!producer_ir || !consumer_ir || !intermediate)
    return fail(SAREK_HIP_E_INVALID_ARG, "fusion_fuse: NULL argument");
  return guarded("fusion_fuse", [&] {
    const ir::Kernel p = ir::parse_kernel(producer_ir), c = ir::parse_kernel(consumer_ir);
    std::optional<ir::Kernel> k;
    switch (mode) {
      case SAREK_HIP_FUSION_VERTICAL: k = fu::fuse(p, c, intermediate); break;
      case SAREK_HIP_FUSION_REDUCTION: k = fu::fuse_reduction(p, c, intermediate); break;
      case SAREK_HIP_FUSION_STENCIL: k = fu::fuse_stencil(p, c, intermediate); break;
      case SAREK_HIP_FUSION_TRY: k = fu::try_fuse(p, c, intermediate); break;
      case SAREK_HIP_FUSION_TRY_ALL: k = fu::try_fuse_all(p, c, intermediate); break;
      default: return fail(SAREK_HIP_E_INVALID_ARG, "fusion_fuse: unknown mode %d", mode);
    }
    if (fused) *fused = k.has_value();
    return deliver(k ? ir::print_kernel(*k) : std::string(), out, out_len, needed, "fusion_fuse");
  });
}

int sarek_hip_fusion_should_fuse(const char *producer_ir, const char *consumer_ir, const char *intermediate,
                                 int *decision, char *reason, size_t reason_len) {
  if (!producer_ir || !consumer_ir || !intermediate || !decision)
    return fail(SAREK_HIP_E_INVALID_ARG, "fusion_should_fuse: NULL argument");
  return guarded("fusion_should_fuse", [&] {
    const fu::Hint h = fu::should_fuse(ir::parse_kernel(producer_ir), ir::parse_kernel(consumer_ir), intermediate);
    *decision = h.decision == fu::Decision::Fuse       ? SAREK_HIP_FUSION_FUSE
                : h.decision == fu::Decision::DontFuse ? SAREK_HIP_FUSION_DONT_FUSE
                                                       : SAREK_HIP_FUSION_MAYBE_FUSE;
    if (reason && reason_len) {
      std::strncpy(reason, h.reason.c_str(), reason_len - 1);
      reason[reason_len - 1] = '\0';
    }
    return static_cast<int>(SAREK_HIP_OK);
  });
}

int sarek_hip_fusion_pipeline(const char *const *kernel_irs, int n_kernels, int automatic, char *out,
                              size_t out_len, size_t *needed, char *report, size_t report_len,
                              size_t *report_needed) {
  return guarded("fusion_pipeline", [&] {
    std::vector<ir::Kernel> kernels;
    if (!read_kernels(kernel_irs, n_kernels, kernels))
      return fail(SAREK_HIP_E_INVALID_ARG, "fusion_pipeline: NULL kernel text");
    ir::Kernel result;
    std::string lines;
    if (automatic) {
      fu::AutoFused r = fu::auto_fuse_pipeline(kernels);
      result = r.kernel;
      for (auto &e : r.eliminated) lines += "eliminated " + e + "\n";
      for (auto &s : r.skipped) lines += "skipped " + s + "\n";
    } else {
      auto r = fu::fuse_pipeline(kernels);
      result = r.first;
      for (auto &e : r.second) lines += "eliminated " + e + "\n";
    }
    int st = deliver(ir::print_kernel(result), out, out_len, needed, "fusion_pipeline");
    int st2 = deliver(lines, report, report_len, report_needed, "fusion_pipeline (report)");
    return st != SAREK_HIP_OK ? st : st2;
  });
}

int sarek_hip_fusion_analyze_pipeline(const char *const *kernel_irs, int n_kernels, char *out, size_t out_len,
                                      size_t *needed) {
  return guarded("fusion_analyze_pipeline", [&] {
    std::vector<ir::Kernel> kernels;
    if (!read_kernels(kernel_irs, n_kernels, kernels))
      return fail(SAREK_HIP_E_INVALID_ARG, "fusion_analyze_pipeline: NULL kernel text");
    return deliver(fu::analyze_pipeline(kernels), out, out_len, needed, "fusion_analyze_pipeline");
  });
}

int sarek_hip_fusion_stencil_info(const char *producer_ir, const char *consumer_ir, const char *intermediate,
                                  int *found, int radii[3], char *inputs, size_t inputs_len, size_t *needed) {
  if (!producer_ir || !consumer_ir || !intermediate || !found || !radii)
    return fail(SAREK_HIP_E_INVALID_ARG, "fusion_stencil_info: NULL argument");
  return guarded("fusion_stencil_info", [&] {
    auto info = fu::analyze_stencil_fusion(ir::parse_kernel(producer_ir), ir::parse_kernel(consumer_ir), intermediate);
    *found = info.has_value();
    std::string names;
    if (info) {
      radii[0] = info->combined_radius;
      radii[1] = info->producer_radius;
      radii[2] = info->consumer_radius;
      for (auto &a : info->input_arrays) names += (names.empty() ? "" : " ") + a;
    }
    return deliver(names, inputs, inputs_len, needed, "fusion_stencil_info");
  });
}

int sarek_hip_fusion_expr_equal(const char *expr_a, const char *expr_b, int *equal) {
  if (!expr_a || !expr_b || !equal) return fail(SAREK_HIP_E_INVALID_ARG, "fusion_expr_equal: NULL argument");
  return guarded("fusion_expr_equal", [&] {
    *equal = fu::expr_equal(ir::parse_expr(expr_a), ir::parse_expr(expr_b));
    return static_cast<int>(SAREK_HIP_OK);
  });
}

int sarek_hip_fusion_subst_array_read(const char *array, const char *index_expr, const char *replacement_expr,
                                      const char *expr, char *out, size_t out_len, size_t *needed) {
  if (!array || !index_expr || !replacement_expr || !expr)
    return fail(SAREK_HIP_E_INVALID_ARG, "fusion_subst_array_read: NULL argument");
  return guarded("fusion_subst_array_read", [&] {
    return deliver(ir::print_expr(fu::subst_array_read(array, ir::parse_expr(index_expr),
                                                       ir::parse_expr(replacement_expr), ir::parse_expr(expr))),
                   out, out_len, needed, "fusion_subst_array_read");
  });
}

int sarek_hip_fusion_detect_reduction(const char *stmt_ir, int *found, char *out, size_t out_len, size_t *needed) {
  if (!stmt_ir || !found) return fail(SAREK_HIP_E_INVALID_ARG, "fusion_detect_reduction: NULL argument");
  return guarded("fusion_detect_reduction", [&] {
    auto r = fu::detect_reduction_pattern(ir::parse_stmt(stmt_ir));
    *found = r.has_value();
    std::string text;
    if (r)
      text = "(reduction " + r->acc.name + " " + std::to_string(r->acc.id) + " " + fu::binop_name(r->op) + " " +
             r->array + " " + r->loop_var.name + " " + std::to_string(r->loop_var.id) + ")";
    return deliver(text, out, out_len, needed, "fusion_detect_reduction");
  });
}

int sarek_hip_fusion_is_reduction_kernel(const char *kernel_ir, const char *array, int *found, char op[8]) {
  if (!kernel_ir || !array || !found) return fail(SAREK_HIP_E_INVALID_ARG, "fusion_is_reduction_kernel: NULL argument");
  return guarded("fusion_is_reduction_kernel", [&] {
    auto r = fu::is_reduction_kernel(ir::parse_kernel(kernel_ir), array);
    *found = r.has_value();
    if (op) {
      std::strncpy(op, r ? fu::binop_name(*r) : "", 7);
      op[7] = '\0';
    }
    return static_cast<int>(SAREK_HIP_OK);
  });
}

}  // extern "C"
