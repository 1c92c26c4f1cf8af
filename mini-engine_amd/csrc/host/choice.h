// Which kernel serves a matrix product of a step: the one table of thresholds in the tree. The native step program
// (program.cpp) and the Python entry point of the products (ops/kernels.py::linear, through me_product_choice) both ask here, so
// the two cannot choose differently. Pure host code: sizes in, a kernel's code out.
#pragma once

#include <stdint.h>

namespace me {

enum ProductKernel {
  kProductF32 = 0,      // the float32 matrix-core product (true 32-bit; the only choice for float32 models)
  kProductSmall = 1,    // the small matrix-core kernel: up to 64 rows, gate as epilogue
  kProductStream = 2,   // the weight-streaming kernel: up to 256 rows, gate as epilogue, k in runs for partial sums
  kProductTiled = 3,    // the LDS-tiled matrix-core kernel, gate as epilogue
  kProductLibrary = 4,  // the GEMM library (with this folder's kernels where it has no algorithm)
};

enum ProductRole {
  kRolePlain = 0,  // a projection inside a part
  kRoleDelta = 1,  // a product whose result only ever is the pending delta of the residual stream
  kRoleHead = 2,   // the logits of the wanted rows (float32 results)
  kRoleDeltaInto = 3,  // as kRoleDelta, by a caller that can let the product add its result into the residual stream itself
};

struct ProductChoice {
  int kernel = kProductLibrary;
  int runs = 1;             // runs of k whose float32 partial sums the next add-and-norm adds up (deltas only)
  bool partial_sums = false;  // the result is float32 [runs, m, n] whatever the model's dtype
  bool gate_after = false;    // the gate is a kernel of its own behind the product
  bool adds_into = false;     // the product adds its result into the float32 residual stream (kRoleDeltaInto only)
};

enum NormFusion {
  kNormAlone = 0,     // the add-and-norm kernel, then the product
  kNormInStream = 1,  // add, norm and product in one launch of the weight-streaming kernel
  kNormInSmall = 2,   // add and norm as the prologue of the small matrix-core kernel
};

enum PendingKind { kPendingNone = 0, kPendingTensor = 1, kPendingParts = 2 };

// dtype, out_dtype: 0 float32, 1 bfloat16. rows_of_w counts gate and up rows of a gated weight. `aligned`: x and the
// weight start at multiples of 16 bytes.
ProductChoice choose_product(int dtype, int role, int m, int rows_of_w, int k, int gated, int out_dtype, int units,
                             bool aligned);
int choose_norm_fusion(int dtype, int m, int rows_of_w, int k, int pending, int units, bool aligned);
// Whether a delta of the residual stream (m rows, n = hidden columns, k) adds itself to the stream and leaves the norm
// behind it to the product after the norm (next_rows_of_w rows of hidden, gated or not): no add-and-norm kernel between.
bool choose_carried_norm(int dtype, int m, int n, int k, int next_rows_of_w, int next_gated, int units, bool aligned);
// Whether the output projection behind a decode attention of m items (n = hidden columns) adds up the attention's splits
// itself, so that no kernel of its own does (sizes that the kernel takes are its own matter: me_attention_out_product_supported).
bool choose_split_sum_in_product(int dtype, int m, int n, bool aligned);

// Limits that the rules above share with the arena's sizing.
constexpr int kSmallMaxRows = 64;      // what the small matrix-core kernel accepts
constexpr int kStreamGroupRows = 256;  // what the weight-streaming kernel accepts, in groups of 64 rows
constexpr int kMaxRuns = 16;           // the most runs of k a delta is cut into

}  // namespace me
