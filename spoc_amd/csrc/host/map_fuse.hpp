// Element-wise kernels recognised as a class and rebuilt in the stream kernels' shape (map_fuse.cpp).
#pragma once
#include <cstdint>
#include <optional>
#include <string>
#include <vector>

#include "ir.hpp"

namespace sarek_hip {
namespace ir {

// out[tid] = f(in_1[tid], ..., in_k[tid], scalars, tid) for tid < n
struct MapKernel {
  struct Param {
    std::string name;
    enum Kind { Vec, F32, I32 } kind = Vec;
  };
  std::vector<Param> params;   // the kernel's parameters in order (a vector is a buffer and its length at a launch)
  int out = -1, n = -1;        // indices into params: the vector written, the bound
  std::vector<int> inputs;     // the vectors read, ascending
  std::string tid;             // name of the thread-id variable
  std::string body;            // HIP statements that set sarek_f_res from <vector>__e, the scalars and tid
  bool is_max = false;         // match_tree: the "take the greater" tree instead of the sum
  std::string pad;             // match_tree, maximum: the fill value of slots past n, as HIP text
};

// The shape above, or nothing: one guarded store under immutable lets, every read at [tid], no mutable state,
// helper functions, records, atomics, barriers or launch-geometry intrinsics in the element's expression.
std::optional<MapKernel> match_map(const Kernel &k);

// HIP source of `sarek_map(<the kernel's parameters without the vector lengths>, float* partials)`: 256-thread
// workgroups of 4096 elements, ceil(n / 4096) of them; reduce = 1 also stores partials[j] = sum of out[256 j .. 256 j + 255]
// in the order of the hand block-256 sum, reduce = 2 their maximum by the tree's comparisons in the tree's order, slots
// past n counting as the value with the bits pad_bits; 0 neither.
std::string map_source(const MapKernel &m, int reduce, bool nt_loads, uint32_t pad_bits = 0);

// The block-256 tree sum (benchmarks/bench_reduction.ml:62-96) with a pure element-wise expression where the
// reference's kernel reads its input (the dot product of bench_dot_product.ml:16-54 is one such): `out` is then the
// vector of block sums, `tid` the global index, `body` the expression's statements.  Nothing when the kernel differs
// from that tree in anything but the expression.
std::optional<MapKernel> match_tree_sum(const Kernel &k);
// The same for the "take the greater" tree of benchmarks/bench_reduction_max.ml:18-100 (any constant fill value).
std::optional<MapKernel> match_tree_max(const Kernel &k);

// HIP source of `sarek_tree(<the kernel's parameters without the vector lengths>)`: 256-thread workgroups of 32
// blocks of 256 elements, sums in the order of the hand block-256 kernel (maxima: the tree's comparisons in the tree's order).
std::string tree_sum_source(const MapKernel &m, bool nt_loads);
std::string tree_max_source(const MapKernel &m);

}  // namespace ir
}  // namespace sarek_hip
