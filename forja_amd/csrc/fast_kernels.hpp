// Specialised gfx950 kernels for the hot shapes of the ragged forward step.  Each `try_fast_*`
// inspects the operand layouts and either enqueues the specialised kernel and returns true, or
// returns false so the caller falls back to the strided generic kernel.
#pragma once

#include <vector>

#include "kernels.hpp"

struct fh_backend;

namespace fh {

// Implemented in backend.cpp.
char *backend_workspace(fh_backend *backend, uint64_t bytes);
// The most backend_workspace can hand out: unbounded, except while the backend takes its scratch
// from the library's fixed array.
uint64_t backend_workspace_limit(fh_backend *backend);
hipStream_t backend_stream(fh_backend *backend);
uint32_t backend_compute_units(fh_backend *backend);
void backend_profile_begin(fh_backend *backend, uint32_t kernel_class);
void backend_profile_end(fh_backend *backend, uint32_t kernel_class);

// Identity of a route plan: the indices view it was packed from and the tiling.
struct RoutePlanKey {
  uint64_t buffer, offset, stride0, stride1;
  uint32_t rows, k, experts, tile;
};
// Device storage (at least `bytes`) for a route plan that outlives its dispatch, so that the two
// routed projections of a layer pack their shared indices once.  `*reuse` is set when the storage
// already holds the plan for `key`: the same indices view, not written since it was packed, in
// the same submission.  Null when allocation fails.
char *backend_route_plan(fh_backend *backend, const RoutePlanKey &key, uint64_t bytes, bool *reuse);

// Identity of an attention work plan: the metadata it was built from (allocation ids and device
// addresses of cu_seqlens, q_starts, activity, tables and generations; the last two because the
// per-token failure flags kept with the plan come from them) and every scalar it depends on.
struct AttentionPlanKey {
  uint64_t buffers[5], address[5];
  uint32_t params[14];
};
// Like backend_route_plan, for the work plan the attention dispatches of one submission share:
// every layer of a step attends with the same lanes, starts and tables.
char *backend_attention_plan(fh_backend *backend, const AttentionPlanKey &key, uint64_t bytes,
                             bool *reuse);

// Brackets one kernel launch with HIP events when profiling is enabled.
struct KernelTimer {
  fh_backend *backend;
  uint32_t kernel_class;
  KernelTimer(fh_backend *b, uint32_t c) : backend(b), kernel_class(c) {
    backend_profile_begin(backend, kernel_class);
  }
  ~KernelTimer() { backend_profile_end(backend, kernel_class); }
};

struct QmmProblem {
  View x, packed, scales, biases, out;
  uint32_t rows, inner, columns, bits, group;
  // Optional [rows, columns] bf16 rows added to the f32 result before it is rounded (the dense
  // residual-add epilogue); only honoured together with a bf16 `out`.
  const View *residual = nullptr;
  // Allocation identities of packed, scales and biases (0: not known): what a kept copy of the
  // prepared weights is watched by.
  uint64_t weight_buffers[3] = {0, 0, 0};
};
bool try_fast_quant_matmul(fh_backend *backend, const QmmProblem &problem);
// The f32 vector-ALU kernel for what the matrix-core kernels do not take: any float activation and
// output dtype, 4- or 8-bit weights, groups of 32/64/128, f16 or bf16 scales, contiguous rows
// (`residual` of any float dtype).  False when the operands do not fit it either.
bool try_valu_quant_matmul(fh_backend *backend, const QmmProblem &problem);

// Its routed forms: the projection out[r,s,:] = x[r,:] . W[indices[r,s]]^T (`weights` null) and
// the weighted sum out[r,:] = sum_s weights[r,s] * (x[r,s,:] . W[indices[r,s]]^T); `out` may be an
// f32 accumulator view.  Same operand conditions; false when they do not hold.
bool try_valu_gather(fh_backend *backend, const View &x, const View &packed, const View &scales,
                     const View &biases, const View &indices, const View *weights, const View &out,
                     uint32_t rows, uint32_t k, uint32_t inner, uint32_t experts, uint32_t columns,
                     uint32_t bits, uint32_t group, ErrorSlot *error);
// Dequantise-once tiled GEMM for many rows; operands as checked by try_fast_quant_matmul.  False
// when the launch could not be configured.  On success `*refused` points at a device word the
// launched kernels leave non-zero when some scale or bias is outside their fp16 scheme; they
// have then written nothing and the caller must run a kernel conditioned on that word.
// `*refused` is null when the weights are known to be inside the scheme (their prepared form is
// kept, see backend_prepared_weights): nothing else need run.  False also when they are known to
// be outside it.
bool launch_quant_gemm(fh_backend *backend, const QmmProblem &problem, const uint32_t **refused);

// The prepared (dequantised, fp16) form of a weight matrix, kept from the first prefill product
// that needs it until one of its three allocations is written or released: a prompt is many
// chunks and a server many prompts, and preparing 2 bytes per weight again for each is a twentieth
// of a large layer's time and a tenth of a small model's.  `bytes` of device memory followed by a
// flag word; *fresh says the caller must fill them (and then report the flag through
// backend_prepared_verdict).  *verdict: -1 not known yet, 0 inside the fp16 scheme, 1 outside it
// (nothing is kept then but the verdict).  Null when nothing can be kept (allocation identities
// unknown, the memory set aside for it used up, a caller that may not allocate).
struct PreparedKey {
  uint64_t buffers[3];
  const void *address[3];
  uint32_t columns, inner;
};
char *backend_prepared_weights(fh_backend *backend, const PreparedKey &key, uint64_t bytes, bool *fresh,
                               int *verdict);
// Waits for the stream and reads the flag word behind the operand the caller has just filled.
void backend_prepared_verdict(fh_backend *backend, const PreparedKey &key);

// ---- qmm_ksplit.hip: products over at most 32 activation rows per weight (decode GEMV, routed
// MoE tiles), K split over the waves of a workgroup with the rows stationary in registers.
// Operands as try_fast_quant_matmul checks them: bf16 rows, 4-bit weights in groups of 64 with
// bf16 scales and biases, aligned contiguous rows.
// Whether K has an instantiation (dense: at most 16 rows for the longest rows; routed: tiles of
// 16 or 32 rows) and the output columns are whole batches of the kernel (32 or 64 columns; 16 or
// 32 per projection of a pair).
bool ksplit_supports(uint32_t inner, uint32_t columns, bool pair, bool routed);
struct KsplitDense {
  const void *x;            // bf16 rows, or f32 rows with `wide`
  uint64_t x_row_stride;
  const uint32_t *packed;
  const uint16_t *scales, *biases;
  void *out;
  uint64_t out_row_stride;
  uint32_t out_f32;
  const void *residual;     // rows of the activations' dtype
  uint64_t residual_row_stride;
  uint32_t rows, inner, columns;
  bool wide;                // f32 activations, residual and result (at most 32 rows)
  // Non-zero: `inner` is a range of the K of weight rows `weight_inner` long; x, packed, scales and
  // biases point at the range's first element.
  uint32_t weight_inner;
};
// Whether launch_ksplit_dense takes a product of `rows` rows: at most 128, in row tiles of 16 or
// 32, and more than one tile only for weights small enough to stay cached between the tiles.
bool ksplit_dense_supports(uint32_t rows, uint32_t inner, uint32_t columns, bool wide = false);
// False when ksplit_dense_supports is: nothing was launched.
bool launch_ksplit_dense(fh_backend *backend, const KsplitDense &problem);
struct KsplitRouted {
  const void *x;            // bf16 rows, or f32 rows with `wide`
  uint64_t x_row_stride;
  const uint32_t *packed[2];
  const uint16_t *scales[2], *biases[2];
  bool pair;                // gate/up pair with SwiGLU (bf16 out), else one projection
  void *out;                // [routes, columns] dense rows, bf16 or f32
  uint32_t out_f32;
  uint32_t inner, columns;
  const uint32_t *sorted_routes, *blocks, *n_blocks;
  uint32_t max_blocks, tile_rows, route_div;
  bool wide;                // f32 activations and results; tiles of 16 routes only
};
bool launch_ksplit_routed(fh_backend *backend, const KsplitRouted &problem);

// A row-wise RMS normalisation the next dispatch applies to the rows a weighted sum produces:
// out[r,:] = rows[r,:] * rsqrt(mean(rows[r,:]^2) + eps) * weight[r,:], everything bf16 or
// everything f32 (`wide`).  The kernel that writes the rows can produce this too and save the launch.
struct NormTail {
  const void *weight;
  void *out;
  uint64_t weight_stride, out_stride;   // elements per row
  float eps;
  bool wide;
};

struct GatherProblem {
  View x;           // projection: [R,K]; weighted sum: [R,k,K]
  View packed[2], scales[2], biases[2];
  View indices;     // [R,k]
  uint64_t indices_buffer;  // allocation identity of `indices`
  View weights;     // weighted sum only: [R,k]
  View out;         // projection: [R,k,N]; weighted sum: [R,N]
  uint32_t rows, k, inner, experts, columns, bits, group;
  // weighted sum only: the normalisation that follows, and where to say that it has been done
  const NormTail *norm_tail;
  bool *norm_tail_taken;
};

// The routes of a gather problem packed by expert on the device (or the plan the previous routed
// dispatch packed from the same indices): `blocks` holds (expert, first, count <= tile) triples over
// `sorted_routes`, `n_blocks[0]` how many; bad routes are left out and reported.  `rest` is `extra`
// bytes of workspace.
struct PackedRoutes {
  const uint32_t *sorted_routes, *blocks, *n_blocks;
  uint32_t max_blocks, tile;
  char *rest;
};
bool pack_routes(fh_backend *backend, const GatherProblem &problem, uint64_t extra, ErrorSlot *error,
                 PackedRoutes *packed);
// out[r,:] = residual? + sum_s weights[r,s] * partial[r*k+s,:] over the valid routes, ascending s.
void launch_combine_routes(hipStream_t stream, const float *partial, const GatherProblem &problem,
                           const View *residual);
// Routed products grouped by expert on the f32 vector ALUs, for batches with several routes per
// expert: `weighted` false computes out[r,s,:] (a dense [R,k,N] view, zero rows for bad routes),
// true the weighted sum with an optional residual.  False when the operands do not fit.
bool try_valu_gather_grouped(fh_backend *backend, const GatherProblem &problem, int projection,
                             const View &out, bool weighted, const View *residual, ErrorSlot *error);
// projections = 1 (plain) or 2 (gate/up pair); swiglu = fuse silu(acc0)*acc1.
bool try_fast_gather_projection(fh_backend *backend, const GatherProblem &problem, int projections,
                                bool swiglu, ErrorSlot *error);
// residual may be null; otherwise out = residual + sum.
bool try_fast_gather_weighted(fh_backend *backend, const GatherProblem &problem,
                              const View *residual, ErrorSlot *error);

struct LaneAttention {
  View q, key_pool, value_pool, table, generations, activity, out;
  uint32_t query_heads, query_length, kv_heads, width, value_width, key_length, query_start;
  float scale;
  bool causal;
  uint32_t page_tokens, physical_pages, logical_pages;
};
bool try_fast_lane_attention(fh_backend *backend, const LaneAttention &lane, ErrorSlot *error);

struct RaggedAttention {
  View q, k_new, v_new, tables, generations, cu_seqlens, q_starts, activity;
  View out, key_pool, value_pool;
  uint32_t tokens, lanes, query_heads, kv_heads, width, value_width, page_tokens, physical_pages,
      table_pages;
  float scale;
  // allocation identities of cu_seqlens, q_starts, activity, tables, generations (0: none)
  uint64_t metadata_buffers[5];
  // A failure of query token t is recorded in error[t * error_stride]: 0 for one dispatch, the
  // distance between the member dispatches' records when a run of per-lane dispatches is fused.
  uint32_t error_stride;
  // ... and failures of the attention proper (as opposed to the append) that many records further
  // on: the position of the attention dispatch within a fused member.
  uint32_t attention_error_offset;
  // The caller vouches that no lane brings more than one query row (checked on the device when
  // the work plan is built; a violation is reported).  The attention kernel can then store a
  // lane's new key and value row itself, because no other row's attention reads them.
  uint32_t one_row_per_lane;
};
// Always handles the problem (specialised kernel when the layout allows, generic otherwise);
// false only when workspace allocation fails.
bool run_ragged_attention(fh_backend *backend, const RaggedAttention &problem, ErrorSlot *error);

// Recognised guest row programs (by canonical expression) and their constants.
enum ProgramKindFast {
  kProgramGeneric = 0, kProgramRmsNorm, kProgramResidualNorm, kProgramQkNormRope,
  kProgramSiluMul, kProgramAdd   // element-wise: in0 * sigmoid(in0) * in1, in0 + in1
};
struct ProgramClass {
  int kind;
  uint32_t axis;  // the axis the program's extent/index instruction names (must be the last)
  float c[4];
};
ProgramClass classify_program(uint32_t kind, const fh_inst *insts, uint32_t n_insts,
                              const uint32_t *pairs, uint32_t n_pairs);
bool try_fast_program(hipStream_t stream, const ProgramClass &cls, const ProgramArgs &args,
                      uint64_t elements);
// Whether the program is the plain RMS normalisation of bf16 or f32 rows of at most 2048 columns
// that norm_rows_kernel would run, reading exactly `produced`; fills `tail` if so.
bool norm_tail_of(const ProgramClass &cls, const ProgramArgs &args, const View &produced,
                  NormTail *tail);
// combine_routes_rows_kernel followed by that normalisation, one workgroup per row: `out` gets
// the sums (+ residual), `tail.out` their normalisation.  columns <= 2048, a multiple of 8;
// routes <= 8; rows of the tail's dtype with 16-byte aligned pieces of 8 elements.
void launch_combine_routes_norm(hipStream_t stream, const float *partial, const View &indices,
                                const View &weights, const void *residual,
                                uint64_t residual_row_stride, void *out, uint64_t out_row_stride,
                                uint32_t rows, uint32_t routes, uint32_t columns, uint32_t experts,
                                const NormTail &tail);

// Epilogue recognisers: `acc + extra` and `silu(acc0) * acc1` in the instruction orders the SDK
// emits (crates/forja-sdk/src/nn/blocks.rs:406-416) and commuted variants.
bool is_add_epilogue(const std::vector<fh_inst> &insts, const std::vector<uint32_t> &pairs);
bool is_swiglu_epilogue(const std::vector<fh_inst> &insts, const std::vector<uint32_t> &pairs);

}  // namespace fh
