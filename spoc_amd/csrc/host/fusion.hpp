// Kernel fusion on the IR: access-pattern analysis, vertical (map -> map), map -> reduce
// and stencil fusion, the fuse / don't-fuse heuristic and the pipeline drivers of
// sarek/sarek/Sarek_fusion.ml, for hosts that hold kernels as IR text and have no OCaml.
#pragma once
#include <optional>
#include <string>
#include <utility>
#include <vector>

#include "ir.hpp"

namespace sarek_hip {
namespace ir {
namespace fusion {

// Sarek_fusion.ml:17-22
struct AccessPattern {
  enum Kind { OneToOne, Stencil, Reduction, Gather, Unknown } kind = Unknown;
  ExprP index;                 // OneToOne
  std::vector<int> offsets;    // Stencil, sorted, unique
  Binop op = Binop::Add;       // Reduction
};

// Sarek_fusion.ml:25-30; both lists are sorted by array name.
struct Info {
  std::vector<std::pair<std::string, AccessPattern>> reads, writes;
  bool has_barriers = false;
  bool has_atomics = false;
};

struct ReductionLoop {         // for i = .. to ..: acc = acc op arr[i]
  Var acc;
  Binop op;
  std::string array;
  Var loop_var;
};

struct StencilFusionInfo {     // Sarek_fusion.ml:821-826
  int combined_radius = 0, producer_radius = 0, consumer_radius = 0;
  std::vector<std::string> input_arrays;
};

enum class Decision { Fuse, DontFuse, MaybeFuse };
struct Hint {
  Decision decision;
  std::string reason;
};

// Fusion_error.Empty_pipeline (sarek/sarek/Fusion_error.ml:15-39); what() is the
// reference's error_to_string text.
struct EmptyPipeline : std::runtime_error {
  using std::runtime_error::runtime_error;
};

bool expr_equal(const ExprP &a, const ExprP &b);
bool expr_uses_array(const std::string &arr, const ExprP &e);
bool stmt_uses_array(const std::string &arr, const StmtP &s);
ExprP subst_array_read(const std::string &arr, const ExprP &idx, const ExprP &replacement, const ExprP &e);
StmtP subst_array_read_stmt(const std::string &arr, const ExprP &idx, const ExprP &replacement, const StmtP &s);
bool has_barrier(const StmtP &s);
Info analyze(const Kernel &k);

bool can_fuse(const Kernel &producer, const Kernel &consumer, const std::string &intermediate);
Kernel fuse(const Kernel &producer, const Kernel &consumer, const std::string &intermediate);
std::pair<Kernel, std::vector<std::string>> fuse_pipeline(const std::vector<Kernel> &kernels);

std::optional<ReductionLoop> detect_reduction_pattern(const StmtP &s);
std::optional<Binop> is_reduction_kernel(const Kernel &k, const std::string &arr);
bool can_fuse_reduction(const Kernel &map, const Kernel &reduce, const std::string &intermediate);
Kernel fuse_reduction(const Kernel &map, const Kernel &reduce, const std::string &intermediate);
std::optional<Kernel> try_fuse(const Kernel &producer, const Kernel &consumer, const std::string &intermediate);

int stencil_radius(const std::vector<int> &offsets);
std::optional<std::vector<int>> get_stencil_info(const Kernel &k, const std::string &arr);
bool can_fuse_stencil(const Kernel &producer, const Kernel &consumer, const std::string &intermediate);
std::optional<StencilFusionInfo> analyze_stencil_fusion(const Kernel &producer, const Kernel &consumer,
                                                        const std::string &intermediate);
Kernel fuse_stencil(const Kernel &producer, const Kernel &consumer, const std::string &intermediate);
std::optional<Kernel> try_fuse_all(const Kernel &producer, const Kernel &consumer,
                                   const std::string &intermediate);

Hint should_fuse(const Kernel &producer, const Kernel &consumer, const std::string &intermediate);
struct AutoFused {
  Kernel kernel;
  std::vector<std::string> eliminated, skipped;   // in the reference's list order (latest first)
};
AutoFused auto_fuse_pipeline(const std::vector<Kernel> &kernels);
std::string analyze_pipeline(const std::vector<Kernel> &kernels);   // the text the reference prints

const char *binop_name(Binop op);        // the IR text's operator word
std::string print_pattern(const AccessPattern &p);
std::string print_info(const Info &info);

}  // namespace fusion
}  // namespace ir
}  // namespace sarek_hip
