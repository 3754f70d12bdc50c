// Program of a fused elementwise region: a small register machine evaluated per
// output element by one kernel.  Built by the lazy-graph evaluator from a chain
// of elementwise primitives; every instruction rounds to the dtype of the node
// it stands for, so the result is bit-identical with node-by-node evaluation.
#pragma once
#include "common.h"

namespace rai {

constexpr int kFusedMaxInstr = 32, kFusedMaxLeaves = 8;

enum FusedKind : uint8_t { FUSED_LEAF = 0, FUSED_CONST = 1, FUSED_UNARY = 2, FUSED_BINARY = 3, FUSED_CAST = 4 };

struct FusedInstr {
  uint8_t kind;
  uint8_t op;     // rai_hip_unary_op / rai_hip_binary_op
  uint8_t dtype;  // dtype of the node: the value is rounded to it
  uint8_t a, b;   // operand registers (LEAF: a = leaf index)
  uint8_t pad[3];
  float param;    // CONST value, UNARY parameter
};

struct FusedProgram {
  int n_instr, n_leaves, rank, out_dtype;
  int64_t numel;
  int64_t shape[RAI_HIP_MAX_RANK];                         // iteration space = contiguous output
  int64_t lstride[kFusedMaxLeaves][RAI_HIP_MAX_RANK];      // element strides of the leaves (0 = broadcast)
  const void *leaf[kFusedMaxLeaves];
  int leaf_dtype[kFusedMaxLeaves];
  void *out;
  FusedInstr instr[kFusedMaxInstr];                        // the last instruction is the output
};

int launch_fused_elementwise(int dev, const FusedProgram &p);

}  // namespace rai
