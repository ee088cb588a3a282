// Host-callable launchers for every kernel in libforja_hip.  Each launcher assumes the caller
// (backend.cpp) has already validated operand shapes; none allocates or synchronises.
#pragma once

#include "common.hpp"

namespace fh {

// Device form of one Program IR instruction: the host validator resolves operand types so the
// interpreter needs no dynamic typing.  ty = value type of operand `a` (0 f32, 1 u32, 2 bool).
struct DInst {
  uint8_t kind, op, ty, pad;
  uint32_t a, b, c;
};

constexpr int kMaxProgramInputs = 8;
constexpr int kMaxProgramOutputs = 4;
constexpr int kMaxReductions = 4;

struct ProgramArgs {
  const DInst *insts;
  uint32_t n_insts;
  uint32_t n_inputs;
  uint32_t n_pairs;
  uint32_t rank;
  uint32_t shape[FH_MAX_RANK];
  uint32_t out_slot[kMaxProgramOutputs];
  uint32_t out_value[kMaxProgramOutputs];
  uint32_t n_reduce;
  uint32_t reduce_at[kMaxReductions];
  View inputs[kMaxProgramInputs];
  View outputs[kMaxProgramOutputs];
};

// ---- generic_ops.hip: strided, any-dtype kernels that follow the reference loop order ----
void launch_copy(hipStream_t s, const View &in, const View &out, uint64_t elements);
void launch_program(hipStream_t s, const ProgramArgs &args, bool row, uint64_t elements);
void launch_quant_matmul_generic(hipStream_t s, const View &x, const View &packed,
                                 const View &scales, const View &biases, const View &out,
                                 uint32_t rows, uint32_t inner, uint32_t columns, uint32_t bits,
                                 uint32_t group);
// projection: out [R,k,N]; `experts` bounds the ids; bad routes give zero rows + error.
void launch_gather_projection_generic(hipStream_t s, const View &x, const View &packed,
                                      const View &scales, const View &biases, const View &indices,
                                      const View &out, uint32_t rows, uint32_t inner,
                                      uint32_t experts, uint32_t columns, uint32_t k,
                                      uint32_t bits, uint32_t group, ErrorSlot *error);
void launch_gather_weighted_generic(hipStream_t s, const View &x, const View &packed,
                                    const View &scales, const View &biases, const View &indices,
                                    const View &weights, const View &out, uint32_t rows,
                                    uint32_t routes, uint32_t inner, uint32_t experts,
                                    uint32_t columns, uint32_t bits, uint32_t group,
                                    ErrorSlot *error);
void launch_top_k(hipStream_t s, const View &in, const View &values, const View &indices,
                  uint32_t rows, uint32_t width, uint32_t k, bool normalize);
void launch_argmax(hipStream_t s, const View &in, const View &out, uint32_t rows, uint32_t width);
void launch_quant_embed(hipStream_t s, const View &packed, const View &scales,
                        const View &biases, const View &ids, const View &out, uint32_t id_count,
                        uint32_t vocab, uint32_t packed_width, uint32_t bits, uint32_t group,
                        ErrorSlot *error);
void launch_matmul(hipStream_t s, const View &left, const View &right, const View &out,
                   uint32_t batches, uint32_t rows, uint32_t inner, uint32_t columns);
void launch_rms_norm(hipStream_t s, const View &in, const View &weight, const View &out,
                     uint32_t rows, uint32_t width, float eps);
void launch_rope(hipStream_t s, const View &in, const View &positions, const View &out,
                 uint32_t rows, uint32_t heads, uint32_t width, float theta);
// ordinary [T, elements] <-> pool [P, pt, elements]; table [Lp,2]; activity may have base null.
void launch_paged_copy(hipStream_t s, const View &ordinary, const View &pool, const View &table,
                       const View &generations, const View &activity, bool into_pages,
                       uint32_t tokens, uint32_t elements, uint32_t start, uint32_t page_tokens,
                       uint32_t physical_pages, uint32_t logical_pages, ErrorSlot *error);
// Generic paged attention for one lane: q [Hq,Sq,D] view, out [Hq,Sq,Dv] view.
void launch_paged_sdpa_generic(hipStream_t s, const View &q, const View &key_pool,
                               const View &value_pool, const View &table,
                               const View &generations, const View &activity, const View &out,
                               uint32_t query_heads, uint32_t query_length, uint32_t kv_heads,
                               uint32_t width, uint32_t value_width, uint32_t key_length,
                               uint32_t query_start, float scale, bool causal,
                               uint32_t page_tokens, uint32_t physical_pages,
                               uint32_t logical_pages, ErrorSlot *error);
void launch_fill_seeded(hipStream_t s, const View &out, uint64_t elements, uint32_t kind,
                        uint64_t seed, uint64_t stream, uint64_t first, float lo, float hi);
void launch_fill_u32(hipStream_t s, uint32_t *ptr, uint64_t count, uint32_t value);
void launch_init_errors(hipStream_t s, ErrorSlot *slots, uint32_t count);

// ---- moe.hip ----
// counts [E], offsets [E+1], sorted_routes [R*k], blocks [max_blocks,3], n_blocks [1].
void launch_route_pack(hipStream_t s, const View &indices, uint32_t rows, uint32_t k,
                       uint32_t experts, uint32_t tile_rows, uint32_t *counts, uint32_t *offsets,
                       uint32_t *sorted_routes, uint32_t *blocks, uint32_t max_blocks,
                       uint32_t *n_blocks, ErrorSlot *error, uint32_t *zero_rows = nullptr,
                       uint32_t zero_row_words = 0);


// ---- sampling.hip: Op::Sample / Op::SampleMasked ----
// Rows are processed by at most kSampleGrid workgroups, each with scratch for one row.
constexpr uint32_t kSampleGrid = 128;
uint64_t sample_scratch_bytes(uint32_t rows, uint32_t width);
// logits [rows, width] (rank-2 view), params u32 [5], allow u32 [ceil(width/32)] contiguous or
// null, out u32 with `rows` elements.  Refused parameters or mask set the error slot.
void launch_sample(hipStream_t s, const View &logits, const View &params, const View *allow,
                   const View &out, uint32_t rows, uint32_t width, uint32_t position,
                   void *scratch, ErrorSlot *error);

// ---- lane_fusion.hip: glue for a run of per-lane attention dispatches executed as one launch ----
// Addresses of up to kLaneChunk lanes, passed by value as kernel arguments.
constexpr uint32_t kLaneChunk = 128;
struct LaneSources {
  const uint32_t *table[kLaneChunk];     // the lane's block table, `table_words` words
  const uint32_t *activity[kLaneChunk];  // the lane's activity word; null: always active
  uint32_t start[kLaneChunk];            // position of the lane's query row
};
struct LaneRows {
  void *first[kLaneChunk];   // where the lane's attended row goes
  void *second[kLaneChunk];  // a second copy of it, or null
};
// Lanes [first, first + count) of `lanes`: tables [lanes, table_words], activity/starts [lanes],
// cu [lanes + 1] (one query row per lane) followed by one word, cleared here, that
// launch_lane_conflict_check raises.
void launch_gather_lane_metadata(hipStream_t s, const LaneSources &sources, uint32_t first,
                                 uint32_t count, uint32_t lanes, uint32_t table_words,
                                 uint32_t *tables, uint32_t *activity, uint32_t *starts,
                                 uint32_t *cu);
// Sets *conflict to 1 when an active lane appends into a slot another active lane attends (the
// gathered arrays of launch_gather_lane_metadata; tables as (page, generation) pairs).  False,
// and nothing launched, when there are more lanes than the check holds in LDS.
bool launch_lane_conflict_check(hipStream_t s, const uint32_t *tables, const uint32_t *activity,
                                const uint32_t *starts, uint32_t lanes, uint32_t table_pages,
                                uint32_t page_tokens, uint32_t *conflict);
// rows: [lanes, row_bytes] contiguous.
void launch_scatter_lane_rows(hipStream_t s, const LaneRows &targets, const void *rows,
                              uint32_t first, uint32_t count, uint32_t row_bytes);

// The same glue for runs whose members bring several query rows (prefill chunks recorded per
// sequence next to decode rows).  Up to kChunkMembers members per launch.
constexpr uint32_t kChunkMembers = 64;
struct ChunkSources {
  const uint32_t *table[kChunkMembers];
  const uint32_t *activity[kChunkMembers];   // null: always active
  uint32_t start[kChunkMembers];             // position of the member's first query row
  uint32_t first_token[kChunkMembers];       // query rows of the members before it
  uint32_t append_record[kChunkMembers];     // error record of the dispatch that stores its rows ...
  uint32_t attention_record[kChunkMembers];  // ... and of the one that attends, from the run's first
};
struct ChunkTargets {
  void *target[2][kChunkMembers];            // where the member's rows go (second: null or a copy)
  uint32_t token_stride[2][kChunkMembers];   // bytes between a member's rows, and between the
  uint32_t head_stride[2][kChunkMembers];    // heads of a row, in each destination
  uint32_t first_token[kChunkMembers + 1];
};
// Members [first, first + count) of `lanes`: as launch_gather_lane_metadata, with cu from the
// members' row counts (cu[lanes] = tokens) and the members' record indices in records[2][lanes].
void launch_gather_chunk_metadata(hipStream_t s, const ChunkSources &sources, uint32_t first,
                                  uint32_t count, uint32_t lanes, uint32_t tokens,
                                  uint32_t table_words, uint32_t *tables, uint32_t *activity,
                                  uint32_t *starts, uint32_t *cu, uint32_t *records);
// Sets *conflict to 1 when an active member stores a row into a slot another active member
// attends.
void launch_chunk_conflict_check(hipStream_t s, const uint32_t *tables, const uint32_t *activity,
                                 const uint32_t *starts, const uint32_t *cu, uint32_t lanes,
                                 uint32_t table_pages, uint32_t page_tokens, uint32_t *conflict);
// rows: [tokens, heads, row_bytes] contiguous; moves the rows of `count` members.
void launch_scatter_chunk_rows(hipStream_t s, const ChunkTargets &targets, const void *rows,
                               uint32_t count, uint32_t heads, uint32_t row_bytes);
// Failures the fused launch recorded per query row (staged[2 * token]: storing the row,
// staged[2 * token + 1]: attending) go to the records of the dispatches they belong to; the
// staged records are cleared for the next run.
void launch_fold_chunk_errors(hipStream_t s, ErrorSlot *staged, ErrorSlot *records_of_run,
                              const uint32_t *cu, const uint32_t *records, uint32_t lanes,
                              uint32_t tokens);

}  // namespace fh
