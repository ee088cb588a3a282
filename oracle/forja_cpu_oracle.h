/*
 * CPU restatement of forja's single-threaded reference backend (crates/forja-cpu) for the
 * ragged continuous-batch forward step.
 *
 * THIS IS TEST INFRASTRUCTURE.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
 * leg may load it.  The shipped library (libforja_hip.so) never links, loads or calls it.
 *
 * Every routine works on *decoded* logical arrays in row-major order, exactly as the reference
 * does after `read()` + `decode()` (crates/forja-cpu/src/lib.rs:141-148, :1790-1809): floats are
 * f32, indices are u32.  Results are f32 and are rounded to the storage dtype with orc_encode
 * (lib.rs:1836-1847).  All arithmetic is sequential f32 with no fused multiply-add (the reference
 * is Rust, which never contracts a*b+c); build with -ffp-contract=off.
 *
 * Pinning (what fixes each routine without running the reference) is listed per function in the
 * .c file and exercised by tests/test_oracle_golden.py.
 */
#ifndef FORJA_CPU_ORACLE_H
#define FORJA_CPU_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes: the discriminants used by the C ABI's fh_status for BackendError
 * (crates/forja-core/src/backend.rs:363-426). */
enum {
  ORC_OK = 0,
  ORC_EXECUTION_FAILED = 4,
  ORC_INVALID_INPUT = 10,
  ORC_INDEX_OUT_OF_RANGE = 12
};

/* dtype codes in wit/compute.wit:4-10 order. */
enum { ORC_F32 = 0, ORC_F16 = 1, ORC_BF16 = 2, ORC_I32 = 3, ORC_U32 = 4 };

/* ---- half 2.7.1 conversions (lib.rs:1796-1805, :1841-1842) ---- */
uint16_t orc_f32_to_bf16(float value);
float orc_bf16_to_f32(uint16_t bits);
uint16_t orc_f32_to_f16(float value);
float orc_f16_to_f32(uint16_t bits);
int orc_decode(const void *source, int dtype, size_t count, float *out);
int orc_encode(const float *source, int dtype, size_t count, void *out);

/* ---- strided views (lib.rs:1736-1788): offsets/strides in elements ---- */
int orc_gather(const uint8_t *source, size_t source_len, int elem_size, int rank,
               const uint32_t *shape, const uint64_t *strides, uint64_t offset, uint8_t *out);
int orc_scatter(uint8_t *target, size_t target_len, int elem_size, int rank, const uint32_t *shape,
                const uint64_t *strides, uint64_t offset, const uint8_t *source);

/* ---- affine group-quantised matmul (lib.rs:914-962, :1277-1310) ---- */
float orc_affine_quant_dot(const float *activation, size_t inner, const uint32_t *packed,
                           const float *scales, const float *biases, size_t packed_row,
                           size_t group_row, size_t group_size, int bits);
int orc_quant_matmul(const float *x, const uint32_t *packed, const float *scales,
                     const float *biases, size_t rows, size_t inner, size_t columns, int bits,
                     size_t group_size, float *out);

/* ---- routed projections (lib.rs:1025-1106, :1108-1204) ----
 * invalid[0] = 1 and invalid[1] = lowest bad expert id when a route names an expert >= experts;
 * the status is still ORC_OK so the caller can write the output first, as the reference does. */
int orc_gather_quant_projection(const float *x, const uint32_t *packed, const float *scales,
                                const float *biases, const uint32_t *indices, size_t rows,
                                size_t inner, size_t experts, size_t columns, size_t k, int bits,
                                size_t group_size, float *out, uint32_t invalid[2]);
int orc_gather_quant_weighted_sum(const float *x, const uint32_t *packed, const float *scales,
                                  const float *biases, const uint32_t *indices,
                                  const float *weights, const float *residual, size_t rows,
                                  size_t routes, size_t inner, size_t experts, size_t columns,
                                  int bits, size_t group_size, float *out, uint32_t invalid[2]);

/* ---- selection (lib.rs:519-608) ---- */
int orc_argmax(const float *values, size_t rows, size_t width, uint32_t *out);
/* Op::Sample / Op::SampleMasked (crates/forja-cpu/src/lib.rs:610-678, 1545-1700).  params:
 * temperature bits, top_k, top_p bits, seed low, seed high.  allow: one bit per column, or null. */
int orc_validate_allow_mask(const uint32_t *allow, size_t words, size_t width);
int orc_top_p_keep(const float *row, size_t width, float temperature, float top_p, size_t *keep);
int orc_sample_row(const float *row, size_t width, const uint32_t params[5], uint32_t position,
                   const uint32_t *allow, uint32_t *out);
int orc_sample(const float *values, size_t rows, size_t width, const uint32_t params[5],
               uint32_t position, const uint32_t *allow, uint32_t *out);
int orc_top_k(const float *values, size_t rows, size_t width, size_t k, int normalize,
              float *out_values, uint32_t *out_indices);

/* ---- MoE route packing.  No CPU counterpart in the reference (it loops routes in place); the
 * behaviour restated here is the closed form of count/plan/arrange_expert_routes
 * (crates/forja-metal/src/quant_matmul.metal:1217-1357): a stable counting sort of route ids
 * r*k+s by expert.  counts[experts], offsets[experts+1], sorted_routes[rows*k] (first
 * offsets[experts] entries valid), blocks[3*max_blocks] = (expert,start,count<=tile_rows).
 * Returns the number of blocks, or a negative status. */
long orc_route_pack(const uint32_t *indices, size_t rows, size_t k, size_t experts,
                    size_t tile_rows, uint32_t *counts, uint32_t *offsets,
                    uint32_t *sorted_routes, uint32_t *blocks, size_t max_blocks,
                    uint32_t invalid[2]);

/* ---- paged storage (crates/forja-core/src/paged.rs:97-163, crates/forja-cpu/src/paged.rs) ---- */
int orc_page_table_from_padded(const uint32_t *entries, size_t logical_pages,
                               const uint32_t *generations, size_t physical_pages);
int orc_page_table_resolve(const uint32_t *entries, size_t logical_pages,
                           const uint32_t *generations, size_t physical_pages,
                           uint32_t logical_page, uint32_t *physical);
/* pool: [physical_pages, page_tokens, row_bytes] raw bytes; rows: [tokens, row_bytes]. */
int orc_paged_copy_in(uint8_t *pool, size_t physical_pages, size_t page_tokens, size_t row_bytes,
                      const uint32_t *entries, size_t logical_pages, const uint32_t *generations,
                      uint64_t start, uint64_t tokens, const uint8_t *rows);
int orc_paged_copy_out(const uint8_t *pool, size_t physical_pages, size_t page_tokens,
                       size_t row_bytes, const uint32_t *entries, size_t logical_pages,
                       const uint32_t *generations, uint64_t start, uint64_t tokens,
                       uint8_t *rows);
/* query f32 [Hq, Sq, D]; pools raw bytes of pool_dtype [P, pt, Hkv, D|Dv]; out f32 [Hq, Sq, Dv]. */
int orc_paged_sdpa(const float *query, const void *key_pool, const void *value_pool,
                   int key_dtype, int value_dtype, size_t physical_pages, size_t page_tokens,
                   const uint32_t *entries, size_t logical_pages, const uint32_t *generations,
                   uint32_t query_heads, uint32_t query_length, uint32_t kv_heads, uint32_t width,
                   uint32_t value_width, uint32_t key_length, uint32_t query_start, float scale,
                   int causal, float *out);

/* ---- scalar programs (crates/forja-cpu/src/interpreter.rs) ---- */
typedef struct {
  uint32_t kind; /* 0 input, 1 const, 2 index, 3 extent, 4 unary, 5 binary, 6 select, 7 cast, 8 reduce */
  uint32_t op;   /* unop / binop / redop / value-type / axis, in wit/compute.wit order */
  uint32_t a, b, c; /* operands; const carries f32 bits in a; input carries the slot in a */
} orc_inst;

typedef struct {
  const void *data; /* f32 or u32 values, one per iteration-space element */
  int is_u32;
} orc_program_input;

int orc_interpret(int program_kind /* 0 map, 1 row */, const orc_inst *insts, size_t inst_count,
                  const uint32_t *outputs /* (slot,value) pairs */, size_t output_pairs,
                  size_t output_count, int rank, const uint32_t *shape,
                  const orc_program_input *inputs, size_t input_count, float *const *out);

/* ---- glue (lib.rs:495-517, :681-710, :748-848) ---- */
int orc_rms_norm(const float *values, const float *weights, size_t rows, size_t width, float eps,
                 float *out);
int orc_rope(float *values, const uint32_t *positions, size_t rows, size_t heads, size_t width,
             float theta);
int orc_quant_embed(const uint32_t *packed, const float *scales, const float *biases,
                    const uint32_t *ids, size_t id_count, size_t vocab, size_t packed_width,
                    int bits, size_t group_size, float *out, uint32_t invalid[2]);
int orc_matmul(const float *left, const float *right, size_t batches, size_t rows, size_t inner,
               size_t columns, float *out);

/* ---- seeded synthetic data (this repository's generator; identical integer arithmetic on the
 * GPU so device-generated pools can be checked against this code) ---- */
uint64_t orc_splitmix64(uint64_t value);
uint64_t orc_stream_u64(uint64_t seed, uint64_t stream, uint64_t index);
void orc_fill_words(uint64_t seed, uint64_t stream, uint64_t first, size_t count, uint32_t *out);
void orc_fill_uniform_bf16(uint64_t seed, uint64_t stream, uint64_t first, size_t count, float lo,
                           float hi, uint16_t *out);
void orc_fill_normal_bf16(uint64_t seed, uint64_t stream, uint64_t first, size_t count,
                          uint16_t *out);
void orc_fill_normal_f32(uint64_t seed, uint64_t stream, uint64_t first, size_t count, float *out);

void orc_set_threads(int threads);

#ifdef __cplusplus
}
#endif
#endif
