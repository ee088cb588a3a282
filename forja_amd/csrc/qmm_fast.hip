// Specialised MLX-4bit affine quantised matmul kernels (dense and routed) for gfx950.
#include "fast_kernels.hpp"

#include <algorithm>
#include <string>

namespace fh {

bool try_fast_quant_matmul(hipStream_t, const QmmProblem &) { return false; }

bool try_fast_gather_projection(fh_backend *, const GatherProblem &, int, bool, ErrorSlot *) {
  return false;
}

bool try_fast_gather_weighted(fh_backend *, const GatherProblem &, const View *, ErrorSlot *) {
  return false;
}

bool try_fast_program(hipStream_t, bool, const ProgramArgs &, uint64_t) { return false; }

namespace {

// Canonical expression string of value `v`: commutative operands are sorted so that equivalent
// instruction orders compare equal.
std::string canonical(const std::vector<fh_inst> &insts, uint32_t v, int depth = 0) {
  if (v >= insts.size() || depth > 16) return "?";
  const fh_inst &inst = insts[v];
  switch (inst.kind) {
  case 0: return "in" + std::to_string(inst.a);
  case 1: return "c" + std::to_string(inst.a);
  case 4: return "u" + std::to_string(inst.op) + "(" + canonical(insts, inst.a, depth + 1) + ")";
  case 5: {
    std::string l = canonical(insts, inst.a, depth + 1), r = canonical(insts, inst.b, depth + 1);
    if ((inst.op == 0 || inst.op == 2) && r < l) std::swap(l, r);
    return "b" + std::to_string(inst.op) + "(" + l + "," + r + ")";
  }
  default: return "?";
  }
}

}  // namespace

bool is_add_epilogue(const std::vector<fh_inst> &insts, const std::vector<uint32_t> &pairs) {
  if (pairs.size() != 2 || pairs[0] != 0) return false;
  return canonical(insts, pairs[1]) == "b0(in0,in1)";
}

bool is_swiglu_epilogue(const std::vector<fh_inst> &insts, const std::vector<uint32_t> &pairs) {
  if (pairs.size() != 2 || pairs[0] != 0) return false;
  std::string e = canonical(insts, pairs[1]);
  // gate * sigmoid(gate) * up, in any association
  return e == "b2(b2(in0,u9(in0)),in1)" || e == "b2(in1,b2(in0,u9(in0)))" ||
         e == "b2(in0,b2(in1,u9(in0)))" || e == "b2(b2(in0,in1),u9(in0))" ||
         e == "b2(u9(in0),b2(in0,in1))" || e == "b2(b2(in1,u9(in0)),in0)";
}

}  // namespace fh
