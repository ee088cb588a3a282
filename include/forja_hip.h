/*
 * forja_hip.h - C ABI of libforja_hip.so, the MI355X (gfx950) execution backend for forja's
 * ragged continuous-batch forward step.
 *
 * The entry points mirror, one for one, the methods a `forja_core::Backend` implementation must
 * provide (crates/forja-core/src/backend.rs:650-984) so that the Rust `forja-hip` crate is a thin
 * shim: plain pointers and sizes, no callbacks, no ownership of caller memory beyond a call.
 * Tensors carry element-unit offsets/strides exactly like `forja_core::Layout`
 * (crates/forja-core/src/layout.rs) and name a backend-owned allocation (`BufferId`,
 * crates/forja-core/src/ops.rs:20-60).
 *
 * Threading: every entry point may be called from any thread; a backend serialises internally
 * (one mutex, one HIP stream), like `CpuBackend`'s `Mutex<AllocationRegistry>`
 * (crates/forja-cpu/src/lib.rs:22-24).  Work submitted earlier is visible to later reads.
 */
#ifndef FORJA_HIP_H
#define FORJA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define FH_API __attribute__((visibility("default")))
#else
#define FH_API
#endif

#define FH_MAX_RANK 8     /* crates/forja-core/src/layout.rs:6 */
#define FH_MAX_INPUTS 12  /* 8 primitive inputs (pair gather) + epilogue extras */
#define FH_MAX_OUTPUTS 4  /* crates/forja-core/src/program.rs:31 */

/* BackendError discriminants, declaration order of crates/forja-core/src/backend.rs:363-426. */
typedef enum fh_status {
  FH_OK = 0,
  FH_QUOTA_EXCEEDED = 1,
  FH_ALLOCATION_FAILED = 2,
  FH_INVALID_DEVICE_WORKING_SET = 3,
  FH_EXECUTION_FAILED = 4,
  FH_DEVICE_EXECUTION_FAILED = 5,
  FH_DEVICE_ERROR_FLAG = 6,
  FH_GPU_PREDICTION_EXCEEDED = 7,
  FH_IMPOSSIBLE_RATE = 8,
  FH_TIMEOUT = 9,
  FH_INVALID_INPUT = 10,
  FH_UNSUPPORTED_OPERATION = 11,
  FH_INDEX_OUT_OF_RANGE = 12
} fh_status;

/* wit/compute.wit:4-10 */
typedef enum fh_dtype { FH_F32 = 0, FH_F16 = 1, FH_BF16 = 2, FH_I32 = 3, FH_U32 = 4 } fh_dtype;

/* `Op` (crates/forja-core/src/ops.rs:163-302).  State ops, dense gather-matmul and contiguous
 * sdpa are outside this backend's path and answer FH_UNSUPPORTED_OPERATION. */
typedef enum fh_op_kind {
  FH_OP_PROGRAM = 1,             /* Op::Program: validated map/row scalar program */
  FH_OP_COPY = 2,                /* Op::Copy */
  FH_OP_PAGED_COPY = 3,          /* Op::PagedCopy{direction,start,page_tokens} */
  FH_OP_RMS_NORM = 4,            /* Op::RmsNorm{eps} */
  FH_OP_ARGMAX = 5,              /* Op::Argmax */
  FH_OP_TOP_K = 6,               /* Op::TopK{k,normalize} */
  FH_OP_ROPE = 7,                /* Op::Rope{theta} */
  FH_OP_QUANT_EMBED = 8,         /* Op::QuantEmbed{bits,group_size} */
  FH_OP_MATMUL = 9,              /* Op::Matmul (rank 2 or 3) */
  FH_OP_QUANT_MATMUL = 10,       /* Op::QuantMatmul{bits,group_size} */
  FH_OP_GATHER_QUANT_MATMUL = 11, /* Op::GatherQuantMatmul: 5, 8 (pair) or 6 (weighted sum) inputs */
  FH_OP_PAGED_SDPA_APPEND = 12,  /* Op::PagedSdpaAppend{scale,q_start,page_tokens} */
  FH_OP_PAGED_SDPA = 13,         /* Op::PagedSdpa{scale,causal,q_start,key_length,page_tokens} */
  /* Op::Sample{position,..} (crates/forja-core/src/ops.rs:202-220; executed as
   * crates/forja-cpu/src/lib.rs:610-642, 1577-1700): inputs logits [.., width] (float) and params
   * u32 [5] = temperature bits, top_k, top_p bits, seed low, seed high, read when the dispatch
   * runs; output u32 with one index per row.  `start` carries the position.  The op's
   * chunk_width / fast_top_k / fast_max_chunks / rejection_rounds are tuning attributes of the
   * Metal kernels, checked by forja-core before a backend sees the dispatch, and do not cross
   * this boundary.  Refused live parameters make fh_wait return FH_INVALID_INPUT. */
  FH_OP_SAMPLE = 14,
  /* Op::SampleMasked (ops.rs:221-236; lib.rs:644-678): a third input allow u32
   * [ceil(width/32)], one bit per column; an empty mask or set padding bits are refused. */
  FH_OP_SAMPLE_MASKED = 15,
  /* --- fused forms with no single-dispatch counterpart in the reference --- */
  /* Packed ragged batch of lanes: append each lane's new K/V rows at its q_start, then causal
   * attention through them.  As-if-serial equivalent of, per lane, two Op::PagedCopy{IntoPages}
   * plus one Op::PagedSdpa (or one Op::PagedSdpaAppend when the lane has one query), the sequence
   * engines record per lane (engines/qwen3-coder/src/lib.rs:917-935).
   *   inputs : q [T,Hq,D], k_new [T,Hkv,D], v_new [T,Hkv,Dv], tables u32 [L,table_pages,2],
   *            generations u32 [P], cu_seqlens u32 [L+1], q_starts u32 [L], activity u32 [L]
   *   outputs: out [T,Hq,Dv], key pool [P,pt,Hkv,D], value pool [P,pt,Hkv,Dv]
   * Precondition, NOT checked for this op: no lane's destination (page, slot) is another lane's
   * destination or lies inside another lane's attended range - what the host's copy-on-write
   * pages guarantee (crates/forja-host/src/lib.rs:5408-5470).  Every append of the batch is
   * performed before every attention, so a batch that breaks it is not the serial sequence.
   * (fh_submit does check it, on the device, before it executes a run of per-lane dispatches
   * this way, and falls back to one dispatch at a time.)  Inactive lanes produce zeros and leave
   * the pools untouched; a cu_seqlens that decreases or passes T is refused on the device (zero
   * rows, pools untouched, the lowest offending lane reported).  `k` = 1 is the recorder's promise that no lane brings more
   * than one query row (a decode batch): the library then stores the new rows from inside the
   * attention kernel.  The promise is checked on the device; a lane that breaks it is reported
   * as FH_DEVICE_ERROR_FLAG with the first offending token as value.  `k` = 0: no promise. */
  FH_OP_PAGED_ATTENTION_RAGGED = 32,
  /* GPU-side token->expert packing on its own, for inspection: input indices u32 [R,k];
   * outputs counts u32 [E], offsets u32 [E+1], sorted_routes u32 [R*k], blocks u32 [B,3]
   * (expert,start,count<=tile_rows; unused blocks are (0xffffffff,0,0)).  `k` holds tile_rows.
   * Behavioural reference: count/plan/arrange_expert_routes
   * (crates/forja-metal/src/quant_matmul.metal:1217-1357). */
  FH_OP_ROUTE_PACK = 33,
  /* Seeded synthetic data written on the device (counter-based, integer arithmetic only, so the
   * CPU oracle reproduces it bit for bit).  output: any contiguous tensor.  `k` = kind
   * (0 random u32 words, 1 uniform [lo,hi) with lo=scale hi=eps, 2 normal(0,1));
   * seed = (q_start | key_length<<32), stream = start, first element index = direction. */
  FH_OP_FILL_SEEDED = 34
} fh_op_kind;

typedef uint64_t fh_buffer;  /* allocation identity; 0 is never valid */
typedef uint64_t fh_program; /* prepared scalar program; 0 = none */

/* `Tensor` = (BufferId, Layout, writable) - crates/forja-core/src/ops.rs:62-160. */
typedef struct fh_tensor {
  fh_buffer buffer;
  uint32_t dtype; /* fh_dtype */
  uint32_t rank;
  uint32_t shape[FH_MAX_RANK];
  uint64_t stride[FH_MAX_RANK]; /* elements */
  uint64_t offset;              /* elements */
} fh_tensor;

/* Program IR, wit/compute.wit:75-141 (same enumerator order). */
typedef struct fh_inst {
  uint32_t kind; /* 0 input,1 const,2 index,3 extent,4 unary,5 binary,6 select,7 cast,8 reduce */
  uint32_t op;   /* unop | binop | redop | value-type | axis */
  uint32_t a, b, c; /* operand ids; input slot in a; const f32 bits in a */
} fh_inst;

/* One recorded `Dispatch` (crates/forja-core/src/ops.rs:445-520).  `inputs` holds the op's
 * primitive inputs followed by `n_extras` epilogue extras, as `Dispatch::inputs()` does. */
typedef struct fh_dispatch {
  uint32_t op; /* fh_op_kind */
  float scale; /* sdpa score multiplier */
  float eps;   /* rms-norm stabiliser */
  float theta; /* rope base */
  uint32_t bits, group_size;
  uint32_t k, normalize;
  uint32_t causal, q_start, key_length, page_tokens;
  uint32_t direction; /* paged copy: 0 into pages, 1 out of pages */
  uint32_t start;
  uint32_t n_inputs, n_outputs;
  fh_program program;  /* FH_OP_PROGRAM */
  fh_program epilogue; /* matmul / quant-matmul / gather-quant-matmul only */
  uint32_t accumulator_count, n_extras;
  fh_tensor inputs[FH_MAX_INPUTS];
  fh_tensor outputs[FH_MAX_OUTPUTS];
} fh_dispatch;

/* BackendError payload (backend.rs:363-426). */
typedef struct fh_error {
  uint32_t code;       /* fh_status */
  uint32_t dispatch;   /* index of the first failing dispatch in the submission */
  uint64_t submission; /* monotonic submission serial */
  uint32_t operation;  /* fh_op_kind that raised a data-dependent flag */
  uint32_t flag;       /* 1 = index/page out of range or stale generation */
  uint32_t value;      /* lowest offending index (expert id, token id or logical page) */
  uint32_t reserved;
} fh_error;

typedef struct fh_device_info {
  char family[64];
  uint64_t total_memory;
  uint64_t lds_bytes;
  uint32_t compute_units;
  uint32_t wavefront;
} fh_device_info;

typedef struct fh_backend fh_backend;
typedef struct fh_submission fh_submission;

/* MetalBackend::new / CpuBackend::new (crates/forja-cpu/src/lib.rs:56).  Fails with
 * FH_DEVICE_EXECUTION_FAILED when no gfx950 device is visible: there is no CPU fallback. */
FH_API fh_status fh_create(int device, fh_backend **out);
FH_API void fh_destroy(fh_backend *backend);

/* Backend::alloc (backend.rs:  `alloc(dtype,&[u32])`; lib.rs:67-86): zero-initialised storage. */
FH_API fh_status fh_alloc(fh_backend *backend, uint64_t bytes, fh_buffer *out);
/* Backend::release (lib.rs:155-161): invalidates the allocation and all views of it. */
FH_API fh_status fh_release(fh_backend *backend, fh_buffer buffer);
/* Backend::import_readonly (lib.rs:1369-1377): copies `len` host bytes into read-only storage. */
FH_API fh_status fh_import(fh_backend *backend, const void *bytes, uint64_t len, fh_buffer *out);
/* Backend::write (lib.rs:113-134): contiguous byte range of a writable allocation. */
FH_API fh_status fh_write(fh_backend *backend, fh_buffer buffer, uint64_t byte_offset, const void *bytes,
                   uint64_t len);
/* Backend::read_buffer_range (lib.rs:1379-1394). */
FH_API fh_status fh_read(fh_backend *backend, fh_buffer buffer, uint64_t byte_offset, void *bytes,
                  uint64_t len);
/* Backend::read (lib.rs:141-148): gathers a strided view into logical row-major bytes. */
FH_API fh_status fh_read_tensor(fh_backend *backend, const fh_tensor *tensor, void *bytes, uint64_t len);
/* Backend::prepare_program (lib.rs:1357-1363) / prepare_epilogue: validates and stores the IR. */
FH_API fh_status fh_prepare_program(fh_backend *backend, uint32_t kind /* 0 map, 1 row */,
                             const fh_inst *insts, uint32_t n_insts,
                             const uint32_t *outputs /* (slot,value) pairs */, uint32_t n_pairs,
                             fh_program *out);
FH_API fh_status fh_release_program(fh_backend *backend, fh_program program);

/* Backend::submit (lib.rs:1419-1516): validates every tensor and operand shape, then enqueues the
 * dispatches in order on the backend's stream.  Returns without waiting. */
FH_API fh_status fh_submit(fh_backend *backend, const fh_dispatch *dispatches, uint32_t count,
                    fh_submission **out);
/* fh_submit for callers that cannot allocate.  It has no counterpart in the reference: it exists
 * for code under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc.  It
 * validates and enqueues the dispatches exactly as fh_submit does, in order, one by one (runs of
 * per-lane attention dispatches are not fused: record FH_OP_PAGED_ATTENTION_RAGGED), but takes all
 * device scratch - error records, typed program instructions, route plans, attention plans,
 * epilogue accumulators, kernel workspace - from a fixed array of FH_STATIC_SCRATCH_BYTES inside
 * the library's device image (one copy per GPU, held until the process ends) and calls no
 * hipMalloc, hipFree, hipHostMalloc or event creation.  Inputs and outputs are the caller's
 * tensors as always.  Limits: at most 8192 dispatches; 36 MiB of kernel workspace, 8 MiB of
 * epilogue accumulators, 1 MiB of route plan, 2 MiB of attention plan, 960 KiB of program
 * instructions per call.  Split-KV attention shortens its split count to fit the workspace; any
 * other need beyond a region fails the call with FH_QUOTA_EXCEEDED, `error->dispatch` naming the
 * dispatch that did not fit (earlier dispatches have run, as when fh_submit stops at a failing
 * dispatch).  `error` not null: the call waits for the work and reports data-dependent failures
 * as fh_wait does.  `error` null: the call returns once the work is enqueued and synchronises
 * nothing.  All calls on one GPU share that GPU's array, which keeps the previous call's
 * contents (what must start clear is cleared by a kernel): calls that overlap on one GPU - two
 * backends on it, or a call whose kernels still run when the next call's kernels start on another
 * stream - race. */
#define FH_STATIC_SCRATCH_BYTES (48ull << 20)
FH_API fh_status fh_submit_static(fh_backend *backend, const fh_dispatch *dispatches, uint32_t count,
                           fh_error *error);
/* Submission::wait / wait_timeout (backend.rs:609-647).  timeout_ns 0 = no deadline. */
FH_API fh_status fh_wait(fh_submission *submission, uint64_t timeout_ns, fh_error *error);
/* Submission::gpu_time: device time between the first and last kernel, in ns (0 before wait). */
FH_API uint64_t fh_gpu_time_ns(fh_submission *submission);
FH_API void fh_submission_free(fh_submission *submission);

/* Backend::submit_profiled_retained (backend.rs:813-857): fh_submit with one device timer
 * around every dispatch it executes.  A run of dispatches executed together (per-lane attention
 * fused into one ragged launch, a weighted sum with the normalisation that follows it) gets one
 * timer.  The timers cost two event records per dispatch on the stream. */
FH_API fh_status fh_submit_profiled(fh_backend *backend, const fh_dispatch *dispatches, uint32_t count,
                             fh_submission **out);
/* One entry of SubmissionProfile::per_dispatch (backend.rs:455-500): device time from the start
 * of the submission to the start and to the end of dispatch `dispatch` (gpu_start, gpu_end); the
 * entry covers `dispatches` consecutive dispatches, more than one when they ran as one group. */
typedef struct fh_dispatch_timing {
  uint32_t dispatch, dispatches;
  uint32_t op; /* fh_op_kind of the first dispatch */
  uint32_t reserved;
  uint64_t start_ns, end_ns;
} fh_dispatch_timing;
/* Submission::profile (backend.rs:609-647).  After fh_wait on a submission made by
 * fh_submit_profiled: copies up to `capacity` entries, in dispatch order, and stores the number
 * there are in *n (0 for a submission made by fh_submit).  FH_INVALID_INPUT before fh_wait. */
FH_API fh_status fh_submission_profile(fh_submission *submission, fh_dispatch_timing *out, uint32_t capacity,
                                uint32_t *n);

/* Backend::device_info / memory_usage. */
FH_API fh_status fh_device_info_get(fh_backend *backend, fh_device_info *out);
/* MemoryUsage::charged_bytes (backend.rs:30-39): every device byte the backend holds - the
 * caller's allocations, the operands kept for prefill products (the fp16 bias columns of weight
 * matrices, kept from a weight's first product of more than 128 rows until the weight is written
 * or released), workspace, epilogue accumulators, route and attention plans, lane scratch. */
FH_API fh_status fh_memory_usage(fh_backend *backend, uint64_t *bytes);
/* Backend::set_memory_limit (backend.rs:683-686): the most the caller's allocations plus the kept
 * operands may take; 0 lifts the limit.  An fh_alloc or fh_import that would pass it first drops
 * the kept operands (products then prepare into workspace again) and fails with
 * FH_QUOTA_EXCEEDED if that is not enough.  The same eviction happens, once, when the device
 * itself runs out of memory. */
FH_API fh_status fh_set_memory_limit(fh_backend *backend, uint64_t bytes);
/* Blocks until all submitted work has finished. */
FH_API fh_status fh_synchronize(fh_backend *backend);

/* Profiling aid: device time in ns spent in `kernel_class` (see fh_kernel_class) since the last
 * fh_profile_reset, measured with HIP events recorded on the backend's stream around each
 * dispatch / kernel launch; `launches` receives the count.  fh_profile_enable level: 0 off,
 * 1 times only the single-kernel classes, 2 also times every dispatch. */
typedef enum fh_kernel_class {
  /* whole dispatches, by op */
  FH_KC_OTHER = 0,
  FH_KC_QMM = 1,       /* FH_OP_QUANT_MATMUL */
  FH_KC_MOE = 2,       /* FH_OP_GATHER_QUANT_MATMUL (packing + grouped matmul + combine) */
  FH_KC_ATTENTION = 3, /* paged attention ops (plan + append + attention + merge) */
  /* single kernels: the launch that dominates each class */
  FH_KC_ATTENTION_KERNEL = 4, /* the ragged attention kernel (decode or prefill form) */
  FH_KC_MOE_KERNEL = 5,       /* the routed quantised-matmul kernel of a gather dispatch */
  FH_KC_QMM_KERNEL = 6,       /* the kernels of one dense quantised product: slab + sum (decode rows),
                                 operand preparation + GEMM (prefill rows), or the streaming kernel */
  FH_KC_COUNT = 7
} fh_kernel_class;
FH_API fh_status fh_profile_enable(fh_backend *backend, int enabled);
/* Restricts the kernel-level timers to the classes whose bit is set (bit i = fh_kernel_class i;
 * all classes by default): every timed launch costs two event records on the stream, so a
 * throughput measurement times only the kernel it reports on. */
FH_API fh_status fh_profile_select(fh_backend *backend, uint32_t class_mask);
/* The kernel-level timers take one launch in `every` of each selected class (1: every launch, the
 * default): the launches of a class do the same work layer after layer, and every timed one
 * costs the stream about 6 us between kernels. */
FH_API fh_status fh_profile_sample(fh_backend *backend, uint32_t every);
FH_API fh_status fh_profile_reset(fh_backend *backend);
FH_API fh_status fh_profile_read(fh_backend *backend, uint32_t kernel_class, uint64_t *nanoseconds,
                          uint64_t *launches);

/* Fusion of per-lane attention dispatches.  The engines record a decode batch as one
 * Op::PagedSdpaAppend per lane and layer (engines/qwen3-coder/src/lib.rs:917-935), or as two
 * Op::PagedCopy{IntoPages} plus one Op::PagedSdpa over a single query row
 * (engines/qwen38/src/attention/batch.rs:37-53), each followed by the Op::Copy of the lane's
 * output row into the packed activation.  fh_submit recognises such a run and
 * executes it as one ragged attention launch with the result serial execution gives; a run it
 * cannot prove independent is executed dispatch by dispatch.  On by default.  The Backend trait
 * has no switch for this (the Metal backend fuses in its encoder,
 * crates/forja-metal/src/encoding.rs): these two calls exist for tests and measurements.
 * fh_fusion_stats reports the runs fused and the dispatches they replaced since creation. */
FH_API fh_status fh_fusion_enable(fh_backend *backend, int enabled);
FH_API fh_status fh_fusion_stats(fh_backend *backend, uint64_t *runs, uint64_t *dispatches);

FH_API const char *fh_version(void);

#ifdef __cplusplus
}
#endif
#endif
