// Host side of libforja_hip: allocation registry, operand validation (the checks of
// crates/forja-core/src/ops.rs:1300-2378 for the ops on the ragged forward step), kernel
// selection and the C ABI declared in include/forja_hip.h.
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <new>
#include <set>
#include <thread>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "fast_kernels.hpp"
#include "kernels.hpp"

namespace fh {

namespace {

struct Allocation {
  char *ptr = nullptr;
  uint64_t bytes = 0;
  bool readonly = false;
};

struct Program {
  uint32_t kind = 0;  // 0 map, 1 row
  std::vector<fh_inst> insts;
  std::vector<uint32_t> pairs;  // (slot, value)
  ProgramClass fast{};          // recognised fused form, if any
  bool add_epilogue = false;    // `accumulator + extra`, recognised when the program is prepared
  bool swiglu_epilogue = false; // `silu(accumulator 0) * accumulator 1`
  uint32_t n_inputs = 0;
  uint32_t n_outputs = 0;
  uint32_t n_reduce = 0;
  // Device instruction arrays keyed by the u32-ness mask of the bound inputs.
  std::map<uint32_t, DInst *> typed;
};

bool is_float(uint32_t dtype) { return dtype == FH_F32 || dtype == FH_F16 || dtype == FH_BF16; }
bool is_half(uint32_t dtype) { return dtype == FH_F16 || dtype == FH_BF16; }

uint64_t element_count(const fh_tensor &t) {
  uint64_t count = 1;
  for (uint32_t axis = 0; axis < t.rank; ++axis) count *= t.shape[axis];
  return count;
}

// Layout::is_contiguous (crates/forja-core/src/layout.rs:292-309): extent-1 axes are ignored.
bool is_contiguous(const fh_tensor &t) {
  uint64_t expected = 1;
  for (int axis = (int)t.rank - 1; axis >= 0; --axis) {
    if (t.shape[axis] == 1) continue;
    if (t.stride[axis] != expected) return false;
    expected *= t.shape[axis];
  }
  return true;
}

bool shape_is(const fh_tensor &t, std::initializer_list<uint32_t> shape) {
  if (t.rank != shape.size()) return false;
  uint32_t axis = 0;
  for (uint32_t extent : shape)
    if (t.shape[axis++] != extent) return false;
  return true;
}

}  // namespace

}  // namespace fh

using namespace fh;

// ---------------------------------------------------------------- fixed scratch (fh_submit_static)
//
// Device memory for callers that cannot allocate.  Every GPU the library runs on holds its own
// copy of this array, at its own address, until the process ends; host code never uses the
// array's name as an address (it is a host-side stand-in) but the pointer hipGetSymbolAddress
// gives for the current device, looked up once per device in fh_create.  The array is cut into
// fixed regions, one per kind of scratch the kernels of fh_submit use.
constexpr uint64_t kStaticErrorBytes = 64ull << 10;       // 8192 dispatch error records
constexpr uint64_t kStaticProgramBytes = 960ull << 10;    // typed instructions of a call's programs
constexpr uint64_t kStaticRoutePlanBytes = 1ull << 20;
constexpr uint64_t kStaticAttentionPlanBytes = 2ull << 20;
constexpr uint64_t kStaticAccumulatorBytes = 8ull << 20;
constexpr uint64_t kStaticWorkspaceBytes = 36ull << 20;
constexpr uint64_t kStaticScratchBytes = kStaticErrorBytes + kStaticProgramBytes +
                                         kStaticRoutePlanBytes + kStaticAttentionPlanBytes +
                                         kStaticAccumulatorBytes + kStaticWorkspaceBytes;
static_assert(kStaticScratchBytes == FH_STATIC_SCRATCH_BYTES, "the header states the size");
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
char *g_scratch_of_device[kMaxDevices] = {};   // the array's address on each device seen so far

// The array's device address on `device`, which must be the current device.
char *static_scratch_address(int device) {
  if (device < 0 || device >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_of_device[device]) {
    void *ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return nullptr;
    g_scratch_of_device[device] = (char *)ptr;
  }
  return g_scratch_of_device[device];
}

// Up to 64 typed instructions by value (1 KB of kernel arguments) into device memory.
struct InstructionChunk {
  DInst v[64];
};
__global__ void upload_instructions_kernel(InstructionChunk chunk, DInst *target, uint32_t count) {
  if (threadIdx.x < count) target[threadIdx.x] = chunk.v[threadIdx.x];
}
void upload_instructions(hipStream_t stream, const DInst *insts, uint32_t count, DInst *target) {
  for (uint32_t first = 0; first < count; first += 64) {
    InstructionChunk chunk{};
    const uint32_t n = std::min<uint32_t>(64, count - first);
    for (uint32_t i = 0; i < n; ++i) chunk.v[i] = insts[first + i];
    upload_instructions_kernel<<<dim3(1), 64, 0, stream>>>(chunk, target + first, n);
  }
}

}  // namespace

struct fh_submission {
  fh_backend *backend = nullptr;
  uint64_t serial = 0;
  uint32_t count = 0;
  uint32_t error_capacity = 0;
  std::vector<uint32_t> ops;
  ErrorSlot *device_errors = nullptr;
  ErrorSlot *host_errors = nullptr;  // pinned
  hipEvent_t start = nullptr, end = nullptr;
  hipEvent_t done = nullptr;   // recorded behind the copy of the error records: this submission's completion
  bool waited = false;
  fh_status result = FH_OK;
  fh_error error{};
  uint64_t gpu_ns = 0;
  // fh_submit_profiled: one pair of events per executed dispatch (or fused group of dispatches),
  // turned into offsets from `start` once the submission has been waited for
  bool profiled = false;
  struct Span {
    uint32_t first, dispatches, op;
    hipEvent_t begin, finish;
  };
  std::vector<Span> spans;
  std::vector<fh_dispatch_timing> timings;
};

struct fh_backend {
  std::mutex mutex;
  int device = 0;
  hipStream_t stream = nullptr;
  hipDeviceProp_t props{};
  std::unordered_map<uint64_t, Allocation> allocations;
  std::unordered_map<uint64_t, Program> programs;
  uint64_t next_id = 1;
  uint64_t next_serial = 1;
  uint64_t used_bytes = 0;
  char *workspace = nullptr;
  uint64_t workspace_bytes = 0;
  // route plan kept between the routed projections of a layer
  char *route_plan = nullptr;
  uint64_t route_plan_bytes = 0;
  bool route_plan_valid = false;
  RoutePlanKey route_plan_key{};
  // attention work plan kept between the layers of a step
  char *attention_plan = nullptr;
  uint64_t attention_plan_bytes = 0;
  bool attention_plan_valid = false;
  AttentionPlanKey attention_plan_key{};
  // profiling
  int profiling = 0;  // 0 off, 1 kernel-level timers, 2 also one timer per dispatch
  uint32_t profile_mask = 0xffffffffu;  // kernel classes the kernel-level timers cover
  uint32_t profile_every = 1;              // kernel-level timers take one launch in this many of a class
  uint32_t profile_seen[FH_KC_COUNT] = {};
  struct Timed {
    hipEvent_t start, end;
    uint32_t kernel_class;
  };
  std::vector<Timed> timed;
  std::vector<hipEvent_t> event_pool;
  std::set<fh_submission *> submissions;  // live submissions owning device resources
  // Recycled per-submission error records (device + pinned host), keyed by capacity.
  struct ErrorBuffers {
    ErrorSlot *device;
    ErrorSlot *host;
    uint32_t capacity;
  };
  std::vector<ErrorBuffers> error_pool;
  std::vector<hipEvent_t> open_timers[FH_KC_COUNT];
  // Pinned staging ring for small host->device writes, so fh_write need not wait for the stream.
  char *ring = nullptr;
  uint64_t ring_bytes = 0, ring_head = 0;
  uint64_t class_ns[FH_KC_COUNT] = {};
  uint64_t class_launches[FH_KC_COUNT] = {};

  // Prepared (fp16) forms of weight matrices kept for the prefill GEMM, see
  // backend_prepared_weights; `prepared_watch` counts, per allocation, the entries built from it.
  struct Prepared {
    PreparedKey key;
    char *operand;
    uint64_t bytes;
    int verdict;
  };
  std::vector<Prepared> prepared;
  std::unordered_map<uint64_t, uint32_t> prepared_watch;
  uint64_t prepared_bytes = 0, prepared_limit = 0;
  // operands whose weights were rewritten while nothing could be freed (fh_submit_static): freed
  // by the next call that may wait for the stream
  std::vector<Prepared> dead_prepared;
  // Backend::set_memory_limit: the most `used_bytes` plus the kept operands may reach (0: no limit)
  uint64_t memory_limit = 0;
  static constexpr uint64_t kPreparedTail = 256;   // the flag word behind an operand, padded
  void unwatch(const Prepared &e) {
    for (uint64_t watched : e.key.buffers) {
      auto it = prepared_watch.find(watched);
      if (it != prepared_watch.end() && --it->second == 0) prepared_watch.erase(it);
    }
  }
  void free_operand(Prepared &e) {   // the stream must be idle
    if (!e.operand) return;
    (void)hipFree(e.operand);
    e.operand = nullptr;
    prepared_bytes -= e.bytes + kPreparedTail;
  }
  void reap_dead_prepared() {   // from entry points that may wait for the stream
    if (dead_prepared.empty() || static_mode) return;
    (void)hipStreamSynchronize(stream);
    for (Prepared &e : dead_prepared) free_operand(e);
    dead_prepared.clear();
  }
  // Frees every kept operand (an allocation failed, or the memory limit is reached): products
  // prepare into the workspace again, or keep a fresh copy later.
  bool evict_prepared() {
    if (static_mode || (prepared.empty() && dead_prepared.empty())) return false;
    (void)hipStreamSynchronize(stream);
    bool freed = false;
    for (Prepared &e : dead_prepared) freed |= e.operand != nullptr, free_operand(e);
    dead_prepared.clear();
    for (size_t i = 0; i < prepared.size();) {
      Prepared &e = prepared[i];
      if (!e.operand) {   // a verdict only: costs nothing, stays
        ++i;
        continue;
      }
      freed = true;
      free_operand(e);
      unwatch(e);
      prepared[i] = prepared.back();
      prepared.pop_back();
    }
    return freed;
  }
  void drop_prepared(uint64_t buffer) {   // the allocation is written or released
    if (prepared_watch.find(buffer) == prepared_watch.end()) return;
    const bool can_wait = !static_mode;
    if (can_wait) (void)hipStreamSynchronize(stream);   // kernels in flight may still read an operand
    for (size_t i = 0; i < prepared.size();) {
      Prepared &e = prepared[i];
      if (e.key.buffers[0] != buffer && e.key.buffers[1] != buffer && e.key.buffers[2] != buffer) {
        ++i;
        continue;
      }
      if (can_wait)
        free_operand(e);
      else if (e.operand)
        dead_prepared.push_back(e);   // still allocated and still counted, until it is reaped
      unwatch(e);
      prepared[i] = prepared.back();
      prepared.pop_back();
    }
  }
  // The normalisation the dispatch after a weighted sum applies to its rows, offered to the sum
  // while it is planned, and whether the sum's kernels have produced it.
  const NormTail *norm_tail = nullptr;
  bool *norm_tail_taken = nullptr;
  // Fusion of runs of per-lane attention dispatches: gathered lane metadata followed by the
  // attended rows, kept between the layers of a step (every layer names the same lanes).
  bool lane_fusion = true;
  char *lane_scratch = nullptr;
  uint64_t lane_scratch_bytes = 0;
  bool lane_metadata_valid = false;
  bool lane_conflict = false;     // verdict of the overlap check for the gathered metadata
  uint32_t *host_flag = nullptr;  // pinned word the verdict is read through
  std::vector<uint64_t> lane_metadata_key;          // what the gathered metadata was built from
  std::unordered_set<uint64_t> lane_metadata_watch; // allocations whose writes invalidate it
  uint64_t fused_runs = 0, fused_dispatches = 0;
  // Scratch taken from the library's fixed device array instead of the heap while
  // fh_submit_static runs: nothing may then be allocated or freed, and a need beyond a region's
  // size fails the dispatch (static_overflow tells that failure from an out-of-memory one).
  bool static_mode = false;
  bool static_overflow = false;
  char *static_scratch = nullptr;        // this device's copy of the array
  ErrorSlot *static_host_errors = nullptr;  // pinned mirror of its error records
  char *static_programs = nullptr;       // typed instructions of the call's programs (bump)
  uint64_t static_programs_used = 0;

  // Makes `ptr` hold at least `bytes` (at least `floor` when it has to be allocated anew).
  bool grow(char *&ptr, uint64_t &have, uint64_t bytes, uint64_t floor) {
    if (bytes <= have) return true;
    if (static_mode) {
      static_overflow = true;
      return false;
    }
    (void)hipStreamSynchronize(stream);
    if (ptr) (void)hipFree(ptr);
    ptr = nullptr;
    have = 0;
    uint64_t want = std::max<uint64_t>(bytes, floor);
    void *fresh = nullptr;
    if (hipMalloc(&fresh, want) != hipSuccess) {
      (void)hipGetLastError();
      // out of memory: the kept operands of the prefill products go first, then once more
      if (!evict_prepared() || hipMalloc(&fresh, want) != hipSuccess) {
        (void)hipGetLastError();
        return false;
      }
    }
    ptr = (char *)fresh;
    have = want;
    return true;
  }
  char *ensure_lane_scratch(uint64_t bytes) {
    if (bytes > lane_scratch_bytes) {
      lane_metadata_valid = false;
      attention_plan_valid = false;
    }
    return grow(lane_scratch, lane_scratch_bytes, bytes, 4ull << 20) ? lane_scratch : nullptr;
  }

  // f32 accumulators handed to an epilogue program; separate from `workspace` because the kernel
  // that fills them may carve its own scratch out of the workspace.
  char *accumulators = nullptr;
  uint64_t accumulator_bytes = 0;
  char *ensure_accumulators(uint64_t bytes) {
    return grow(accumulators, accumulator_bytes, bytes, 16ull << 20) ? accumulators : nullptr;
  }
  char *ensure_workspace(uint64_t bytes) {
    return grow(workspace, workspace_bytes, bytes, 64ull << 20) ? workspace : nullptr;
  }
};

namespace {

// Backends that are still alive.  A submission may outlive its backend (a host-language object
// finalised late); it must then release only its own host memory.
std::mutex g_live_mutex;
std::set<fh_backend *> g_live_backends;

bool backend_alive(fh_backend *b) {
  std::lock_guard<std::mutex> lock(g_live_mutex);
  return g_live_backends.count(b) != 0;
}

#define FH_REQUIRE(cond)              \
  do {                                \
    if (!(cond)) return FH_INVALID_INPUT; \
  } while (0)

// Resolves a tensor to a device view after checking identity and that the touched span fits the
// allocation (AllocationRegistry::validate, backend.rs:315-339; Layout::new, layout.rs:203-227).
fh_status make_view(fh_backend *b, const fh_tensor &t, bool writable, View *out) {
  auto it = b->allocations.find(t.buffer);
  FH_REQUIRE(it != b->allocations.end());
  FH_REQUIRE(t.rank <= FH_MAX_RANK && t.dtype <= FH_U32);
  if (writable) FH_REQUIRE(!it->second.readonly);
  uint64_t span = t.offset;
  bool empty = false;
  for (uint32_t axis = 0; axis < t.rank; ++axis) {
    if (t.shape[axis] == 0) {
      empty = true;
      break;
    }
    uint64_t reach = (uint64_t)(t.shape[axis] - 1) * t.stride[axis];
    FH_REQUIRE(t.stride[axis] == 0 || reach / t.stride[axis] == (uint64_t)(t.shape[axis] - 1));
    FH_REQUIRE(span + reach >= span);
    span += reach;
  }
  if (!empty) {
    uint64_t size = dtype_size(t.dtype);
    FH_REQUIRE(span < (1ull << 60));
    FH_REQUIRE((span + 1) * size <= it->second.bytes);
  } else {
    FH_REQUIRE(t.offset * dtype_size(t.dtype) <= it->second.bytes);
  }
  out->base = it->second.ptr;
  out->dtype = t.dtype;
  out->rank = t.rank;
  for (uint32_t axis = 0; axis < FH_MAX_RANK; ++axis) {
    out->shape[axis] = axis < t.rank ? t.shape[axis] : 1;
    out->stride[axis] = axis < t.rank ? t.stride[axis] : 0;
  }
  out->offset = t.offset;
  return FH_OK;
}

// byte_ranges_overlap (crates/forja-core/src/layout.rs:496-560): a conservative span test refined
// by a lattice proof for the common case of two boxes cut from one parent layout (identical
// strides that divide each other): there the offsets decompose into parent coordinates uniquely
// and the boxes overlap iff their intervals overlap on every axis.
bool may_overlap(const fh_tensor &a, const fh_tensor &b) {
  if (a.buffer != b.buffer) return false;
  auto span_of = [](const fh_tensor &t, uint64_t *lo, uint64_t *hi) {
    uint64_t reach = t.offset;
    for (uint32_t axis = 0; axis < t.rank; ++axis) {
      if (t.shape[axis] == 0) {
        *lo = *hi = 0;
        return;
      }
      reach += (uint64_t)(t.shape[axis] - 1) * t.stride[axis];
    }
    *lo = t.offset * dtype_size(t.dtype);
    *hi = (reach + 1) * dtype_size(t.dtype);
  };
  uint64_t alo, ahi, blo, bhi;
  span_of(a, &alo, &ahi);
  span_of(b, &blo, &bhi);
  if (alo == ahi || blo == bhi) return false;
  if (ahi <= blo || bhi <= alo) return false;
  if (a.rank != b.rank || dtype_size(a.dtype) != dtype_size(b.dtype) || a.rank == 0) return true;
  // Axes sorted by descending stride; identical strides required.
  uint32_t order[FH_MAX_RANK];
  for (uint32_t i = 0; i < a.rank; ++i) {
    if (a.stride[i] != b.stride[i] || a.stride[i] == 0) return true;
    order[i] = i;
  }
  std::sort(order, order + a.rank, [&](uint32_t l, uint32_t r) { return a.stride[l] > a.stride[r]; });
  uint64_t ra = a.offset, rb = b.offset;
  bool disjoint = false;
  for (uint32_t n = 0; n < a.rank; ++n) {
    uint32_t axis = order[n];
    uint64_t stride = a.stride[axis];
    uint64_t pa = ra / stride, pb = rb / stride;
    ra %= stride;
    rb %= stride;
    if (n > 0) {
      uint64_t outer = a.stride[order[n - 1]];
      if (outer % stride != 0) return true;
      uint64_t extent = outer / stride;
      if (pa + a.shape[axis] > extent || pb + b.shape[axis] > extent) return true;
    }
    if (pa + a.shape[axis] <= pb || pb + b.shape[axis] <= pa) disjoint = true;
  }
  if (ra != 0 || rb != 0) return true;
  return !disjoint;
}

View null_view() {
  View v{};
  v.base = nullptr;
  return v;
}

// ---------------------------------------------------------------- scalar programs

// Type inference and the structural rules of Program::validate
// (crates/forja-core/src/program.rs): SSA order, typed operands, reductions only in row
// programs and at most four, f32 outputs.  `u32_mask` bit i = input slot i is bound to a u32
// tensor.  Produces the typed device instructions.
constexpr uint32_t kMaxProgramInsts = 256;   // crates/forja-core/src/program.rs:25-31

fh_status type_program(const Program &p, uint32_t u32_mask, uint32_t rank,
                       DInst *out /* [p.insts.size()] */) {
  FH_REQUIRE(p.insts.size() <= kMaxProgramInsts);
  uint8_t types[kMaxProgramInsts];
  uint32_t reductions = 0;
  for (size_t i = 0; i < p.insts.size(); ++i) {
    const fh_inst &in = p.insts[i];
    DInst d{};
    d.kind = (uint8_t)in.kind;
    d.op = (uint8_t)in.op;
    d.a = in.a;
    d.b = in.b;
    d.c = in.c;
    auto operand_ok = [&](uint32_t v) { return (size_t)v < i; };
    switch (in.kind) {
    case 0:
      FH_REQUIRE(in.a < kMaxProgramInputs && in.a < p.n_inputs);
      types[i] = (u32_mask >> in.a) & 1u ? 1 : 0;
      break;
    case 1: types[i] = 0; break;
    case 2:
    case 3:
      FH_REQUIRE(in.op < rank);
      types[i] = 1;
      break;
    case 4:
      FH_REQUIRE(in.op <= 13 && operand_ok(in.a) && types[in.a] == 0);
      types[i] = 0;
      break;
    case 5: {
      FH_REQUIRE(in.op <= 12 && operand_ok(in.a) && operand_ok(in.b));
      uint8_t ta = types[in.a], tb = types[in.b];
      FH_REQUIRE(ta == tb && ta != 2);
      if (ta == 1) FH_REQUIRE(in.op != 3 && in.op != 6);
      d.ty = ta;
      types[i] = in.op >= 7 ? 2 : ta;
      break;
    }
    case 6:
      FH_REQUIRE(operand_ok(in.a) && operand_ok(in.b) && operand_ok(in.c));
      FH_REQUIRE(types[in.a] == 2 && types[in.b] == types[in.c]);
      types[i] = types[in.b];
      break;
    case 7:
      FH_REQUIRE(in.op <= 2 && operand_ok(in.a));
      d.ty = types[in.a];
      types[i] = (uint8_t)in.op;
      break;
    case 8:
      FH_REQUIRE(p.kind == 1 && in.op <= 2 && operand_ok(in.a) && types[in.a] == 0);
      FH_REQUIRE(++reductions <= kMaxReductions);
      types[i] = 0;
      break;
    default: return FH_INVALID_INPUT;
    }
    if (in.kind == 4) d.ty = 0;
    out[i] = d;
  }
  for (size_t pair = 0; pair + 1 < p.pairs.size(); pair += 2) {
    FH_REQUIRE(p.pairs[pair] < p.n_outputs && p.pairs[pair + 1] < p.insts.size());
    FH_REQUIRE(types[p.pairs[pair + 1]] == 0);
  }
  return FH_OK;
}

// Binds a prepared program to tensors (BoundProgram, program.rs:759-857): every input and output
// has exactly the iteration shape; inputs float or u32; outputs float.
fh_status bind_program(fh_backend *b, Program &p, const fh_tensor *inputs, uint32_t n_inputs,
                       const View *input_views, const fh_tensor *outputs, uint32_t n_outputs,
                       const View *output_views, const uint32_t *shape, uint32_t rank,
                       ProgramArgs *args) {
  FH_REQUIRE(n_inputs == p.n_inputs && n_outputs == p.n_outputs);
  FH_REQUIRE(rank >= 1 && rank <= FH_MAX_RANK);
  uint32_t mask = 0;
  for (uint32_t i = 0; i < n_inputs; ++i) {
    FH_REQUIRE(inputs[i].rank == rank);
    for (uint32_t axis = 0; axis < rank; ++axis) FH_REQUIRE(inputs[i].shape[axis] == shape[axis]);
    FH_REQUIRE(is_float(inputs[i].dtype) || inputs[i].dtype == FH_U32);
    if (inputs[i].dtype == FH_U32) mask |= 1u << i;
  }
  for (uint32_t i = 0; i < n_outputs; ++i) {
    FH_REQUIRE(outputs[i].rank == rank && is_float(outputs[i].dtype));
    for (uint32_t axis = 0; axis < rank; ++axis) FH_REQUIRE(outputs[i].shape[axis] == shape[axis]);
  }
  auto cached = p.typed.find(mask | (rank << 16));
  DInst *device = nullptr;
  if (cached != p.typed.end()) {
    device = cached->second;
  } else {
    DInst typed[kMaxProgramInsts];
    fh_status status = type_program(p, mask, rank, typed);
    if (status != FH_OK) return status;
    const uint64_t bytes = p.insts.size() * sizeof(DInst);
    if (b->static_mode) {
      // Nothing may be allocated: the instructions travel as kernel arguments into the call's
      // share of the fixed scratch array and are not kept.  (During validation, before the
      // regions are set up, only the typing is checked.)
      if (b->static_programs) {
        const uint64_t need = (bytes + 255) / 256 * 256;
        if (b->static_programs_used + need > kStaticProgramBytes) {
          b->static_overflow = true;
          return FH_ALLOCATION_FAILED;
        }
        device = (DInst *)(b->static_programs + b->static_programs_used);
        b->static_programs_used += need;
        upload_instructions(b->stream, typed, (uint32_t)p.insts.size(), device);
      }
    } else {
      void *ptr = nullptr;
      if (hipMalloc(&ptr, bytes) != hipSuccess) return FH_ALLOCATION_FAILED;
      if (hipMemcpy(ptr, typed, bytes, hipMemcpyHostToDevice) != hipSuccess)
        return FH_DEVICE_EXECUTION_FAILED;
      device = (DInst *)ptr;
      p.typed[mask | (rank << 16)] = device;
    }
  }
  memset(args, 0, sizeof(*args));
  args->insts = device;
  args->n_insts = (uint32_t)p.insts.size();
  args->n_inputs = n_inputs;
  args->rank = rank;
  for (uint32_t axis = 0; axis < FH_MAX_RANK; ++axis) args->shape[axis] = axis < rank ? shape[axis] : 1;
  args->n_pairs = (uint32_t)(p.pairs.size() / 2);
  FH_REQUIRE(args->n_pairs <= kMaxProgramOutputs);
  for (uint32_t pair = 0; pair < args->n_pairs; ++pair) {
    args->out_slot[pair] = p.pairs[2 * pair];
    args->out_value[pair] = p.pairs[2 * pair + 1];
  }
  args->n_reduce = 0;
  for (uint32_t i = 0; i < p.insts.size(); ++i)
    if (p.insts[i].kind == 8) args->reduce_at[args->n_reduce++] = i;
  for (uint32_t i = 0; i < n_inputs; ++i) args->inputs[i] = input_views[i];
  for (uint32_t i = 0; i < n_outputs; ++i) args->outputs[i] = output_views[i];
  return FH_OK;
}

// ---------------------------------------------------------------- per-op planning

struct Planned {
  const fh_dispatch *d;
  View in[FH_MAX_INPUTS];
  View out[FH_MAX_OUTPUTS];
};

fh_tensor f32_like(const fh_tensor &t) {
  // A contiguous f32 tensor of the same shape (buffer filled in by the caller's view).
  fh_tensor r = t;
  r.dtype = FH_F32;
  uint64_t stride = 1;
  for (int axis = (int)t.rank - 1; axis >= 0; --axis) {
    r.stride[axis] = stride;
    stride *= t.shape[axis];
  }
  r.offset = 0;
  return r;
}

View contiguous_view(char *base, uint32_t dtype, const fh_tensor &like) {
  View v{};
  v.base = base;
  v.dtype = dtype;
  v.rank = like.rank;
  uint64_t stride = 1;
  for (uint32_t axis = 0; axis < FH_MAX_RANK; ++axis) {
    v.shape[axis] = 1;
    v.stride[axis] = 0;
  }
  for (int axis = (int)like.rank - 1; axis >= 0; --axis) {
    v.shape[axis] = like.shape[axis];
    v.stride[axis] = stride;
    stride *= like.shape[axis];
  }
  v.offset = 0;
  return v;
}

// check_quantized_weights (ops.rs:1798-1842 and check_quantized_expert_weights): packed u32
// [.., N, K*bits/32], scales/biases half [.., N, K/group], same dtype.
fh_status check_quant_triple(const fh_tensor &packed, const fh_tensor &scales,
                             const fh_tensor &biases, uint32_t rank, uint32_t inner,
                             uint32_t bits, uint32_t group, uint32_t *columns,
                             uint32_t *experts) {
  FH_REQUIRE(bits == 4 || bits == 8);
  FH_REQUIRE(group == 32 || group == 64 || group == 128);
  FH_REQUIRE(inner != 0 && inner % group == 0);
  FH_REQUIRE(packed.dtype == FH_U32 && packed.rank == rank);
  FH_REQUIRE(is_half(scales.dtype) && biases.dtype == scales.dtype);
  FH_REQUIRE(scales.rank == rank && biases.rank == rank);
  uint32_t n = packed.shape[rank - 2];
  FH_REQUIRE((uint64_t)packed.shape[rank - 1] * 32 == (uint64_t)inner * bits);
  for (const fh_tensor *t : {&scales, &biases}) {
    FH_REQUIRE(t->shape[rank - 2] == n && t->shape[rank - 1] == inner / group);
    if (rank == 3) FH_REQUIRE(t->shape[0] == packed.shape[0]);
  }
  *columns = n;
  if (experts) *experts = rank == 3 ? packed.shape[0] : 1;
  return FH_OK;
}

fh_status run_epilogue(fh_backend *b, const Planned &pl, uint32_t primitive_inputs,
                       char *accumulators, uint32_t accumulator_count) {
  const fh_dispatch &d = *pl.d;
  auto it = b->programs.find(d.epilogue);
  FH_REQUIRE(it != b->programs.end());
  Program &p = it->second;
  FH_REQUIRE(p.kind == 0);
  FH_REQUIRE(d.accumulator_count == accumulator_count);
  FH_REQUIRE(primitive_inputs + d.n_extras == d.n_inputs);
  uint32_t n_inputs = accumulator_count + d.n_extras;
  FH_REQUIRE(n_inputs <= kMaxProgramInputs);
  fh_tensor tensors[kMaxProgramInputs];
  View views[kMaxProgramInputs];
  const fh_tensor &out = d.outputs[0];
  uint64_t elements = element_count(out);
  for (uint32_t i = 0; i < accumulator_count; ++i) {
    tensors[i] = f32_like(out);
    views[i] = contiguous_view(accumulators + (uint64_t)i * elements * 4, FH_F32, out);
  }
  for (uint32_t i = 0; i < d.n_extras; ++i) {
    tensors[accumulator_count + i] = d.inputs[primitive_inputs + i];
    views[accumulator_count + i] = pl.in[primitive_inputs + i];
  }
  ProgramArgs args;
  fh_status status = bind_program(b, p, tensors, n_inputs, views, &out, 1, &pl.out[0], out.shape,
                                  out.rank, &args);
  if (status != FH_OK) return status;
  launch_program(b->stream, args, false, elements);
  return FH_OK;
}

fh_status plan_copy(fh_backend *b, const Planned &pl, bool execute) {
  const fh_dispatch &d = *pl.d;
  FH_REQUIRE(d.n_inputs == 1 && d.n_outputs == 1);
  const fh_tensor &in = d.inputs[0], &out = d.outputs[0];
  FH_REQUIRE(in.rank == out.rank);
  for (uint32_t axis = 0; axis < in.rank; ++axis) FH_REQUIRE(in.shape[axis] == out.shape[axis]);
  bool in_int = in.dtype == FH_I32 || in.dtype == FH_U32;
  bool out_int = out.dtype == FH_I32 || out.dtype == FH_U32;
  FH_REQUIRE(in_int == out_int);
  if (in_int) FH_REQUIRE(in.dtype == out.dtype);
  if (execute) launch_copy(b->stream, pl.in[0], pl.out[0], element_count(out));
  return FH_OK;
}

fh_status plan_program(fh_backend *b, const Planned &pl, bool execute) {
  const fh_dispatch &d = *pl.d;
  auto it = b->programs.find(d.program);
  FH_REQUIRE(it != b->programs.end());
  FH_REQUIRE(d.n_outputs >= 1 && d.n_outputs <= kMaxProgramOutputs);
  FH_REQUIRE(d.n_inputs <= kMaxProgramInputs);
  const fh_tensor &first = d.outputs[0];
  ProgramArgs args;
  fh_status status = bind_program(b, it->second, d.inputs, d.n_inputs, pl.in, d.outputs,
                                  d.n_outputs, pl.out, first.shape, first.rank, &args);
  if (status != FH_OK) return status;
  uint64_t elements = element_count(first);
  if (it->second.kind == 1) FH_REQUIRE(first.shape[first.rank - 1] != 0);
  if (execute) {
    if (try_fast_program(b->stream, it->second.fast, args, elements)) return FH_OK;
    launch_program(b->stream, args, it->second.kind == 1, elements);
  }
  return FH_OK;
}

fh_status plan_quant_matmul(fh_backend *b, const Planned &pl, ErrorSlot *, bool execute) {
  const fh_dispatch &d = *pl.d;
  uint32_t primitive = 4;
  FH_REQUIRE(d.n_outputs == 1 && d.n_inputs == primitive + (d.epilogue ? d.n_extras : 0));
  const fh_tensor &x = d.inputs[0], &out = d.outputs[0];
  FH_REQUIRE(is_float(x.dtype) && out.dtype == x.dtype);
  FH_REQUIRE(x.rank == 2 && out.rank == 2);
  uint32_t rows = x.shape[0], inner = x.shape[1], columns = 0;
  fh_status status = check_quant_triple(d.inputs[1], d.inputs[2], d.inputs[3], 2, inner, d.bits,
                                        d.group_size, &columns, nullptr);
  if (status != FH_OK) return status;
  FH_REQUIRE(shape_is(out, {rows, columns}));
  if (!execute) return FH_OK;
  if (rows == 0 || columns == 0) return FH_OK;
  if (!d.epilogue) {
    QmmProblem problem{pl.in[0], pl.in[1], pl.in[2], pl.in[3], pl.out[0], rows, inner, columns,
                       d.bits, d.group_size};
    for (int i = 0; i < 3; ++i) problem.weight_buffers[i] = d.inputs[1 + i].buffer;
    if (try_fast_quant_matmul(b, problem) || try_valu_quant_matmul(b, problem)) return FH_OK;
    launch_quant_matmul_generic(b->stream, pl.in[0], pl.in[1], pl.in[2], pl.in[3], pl.out[0], rows,
                                inner, columns, d.bits, d.group_size);
    return FH_OK;
  }
  // Recognised epilogue: out = accumulator + extra (the residual add after a dense projection).
  auto prog = b->programs.find(d.epilogue);
  FH_REQUIRE(prog != b->programs.end());
  if (d.accumulator_count == 1 && d.n_extras == 1 &&
      prog->second.add_epilogue && shape_is(d.inputs[primitive], {rows, columns})) {
    QmmProblem fused{pl.in[0], pl.in[1], pl.in[2], pl.in[3], pl.out[0], rows, inner, columns,
                     d.bits, d.group_size, &pl.in[primitive]};
    for (int i = 0; i < 3; ++i) fused.weight_buffers[i] = d.inputs[1 + i].buffer;
    if (try_fast_quant_matmul(b, fused) || try_valu_quant_matmul(b, fused)) return FH_OK;
  }
  // The accumulators live apart from the workspace, which the product kernels use themselves.
  uint64_t elements = (uint64_t)rows * columns;
  char *acc = b->ensure_accumulators(elements * 4);
  if (!acc) return FH_ALLOCATION_FAILED;
  View acc_view = contiguous_view(acc, FH_F32, out);
  QmmProblem problem{pl.in[0], pl.in[1], pl.in[2], pl.in[3], acc_view, rows, inner, columns,
                     d.bits, d.group_size};
  if (!try_fast_quant_matmul(b, problem) && !try_valu_quant_matmul(b, problem))
    launch_quant_matmul_generic(b->stream, pl.in[0], pl.in[1], pl.in[2], pl.in[3], acc_view, rows,
                                inner, columns, d.bits, d.group_size);
  return run_epilogue(b, pl, primitive, acc, 1);
}

fh_status plan_gather(fh_backend *b, const Planned &pl, ErrorSlot *error, bool execute) {
  const fh_dispatch &d = *pl.d;
  FH_REQUIRE(d.n_outputs == 1);
  uint32_t extras = d.epilogue ? d.n_extras : 0;
  FH_REQUIRE(d.n_inputs >= extras);
  uint32_t primitive = d.n_inputs - extras;
  FH_REQUIRE(primitive == 5 || primitive == 6 || primitive == 8);
  const fh_tensor &x = d.inputs[0], &out = d.outputs[0];
  FH_REQUIRE(is_float(x.dtype) && out.dtype == x.dtype);
  uint32_t columns = 0, experts = 0;
  if (primitive == 6) {
    // check_gather_quant_weighted_sum (ops.rs:1884-1931)
    const fh_tensor &idx = d.inputs[4], &w = d.inputs[5];
    FH_REQUIRE(x.rank == 3 && x.shape[1] != 0);
    FH_REQUIRE(w.dtype == x.dtype && idx.dtype == FH_U32);
    uint32_t rows = x.shape[0], routes = x.shape[1], inner = x.shape[2];
    fh_status status = check_quant_triple(d.inputs[1], d.inputs[2], d.inputs[3], 3, inner, d.bits,
                                          d.group_size, &columns, &experts);
    if (status != FH_OK) return status;
    FH_REQUIRE(shape_is(idx, {rows, routes}) && shape_is(w, {rows, routes}));
    FH_REQUIRE(shape_is(out, {rows, columns}));
    FH_REQUIRE(experts <= 4096);
    if (!execute || rows == 0 || columns == 0) return FH_OK;
    bool fuse_residual = false;
    GatherProblem problem{};
    problem.x = pl.in[0];
    problem.packed[0] = pl.in[1];
    problem.scales[0] = pl.in[2];
    problem.biases[0] = pl.in[3];
    problem.indices = pl.in[4];
    problem.indices_buffer = d.inputs[4].buffer;
    problem.weights = pl.in[5];
    problem.rows = rows;
    problem.k = routes;
    problem.inner = inner;
    problem.experts = experts;
    problem.columns = columns;
    problem.bits = d.bits;
    problem.group = d.group_size;
    problem.norm_tail = b->norm_tail;
    problem.norm_tail_taken = b->norm_tail_taken;
    if (!d.epilogue) {
      problem.out = pl.out[0];
      if (try_fast_gather_weighted(b, problem, nullptr, error)) return FH_OK;
      if (try_valu_gather_grouped(b, problem, 0, pl.out[0], true, nullptr, error)) return FH_OK;
      if (try_valu_gather(b, pl.in[0], pl.in[1], pl.in[2], pl.in[3], pl.in[4], &pl.in[5], pl.out[0], rows,
                          routes, inner, experts, columns, d.bits, d.group_size, error))
        return FH_OK;
      launch_gather_weighted_generic(b->stream, pl.in[0], pl.in[1], pl.in[2], pl.in[3], pl.in[4],
                                     pl.in[5], pl.out[0], rows, routes, inner, experts, columns,
                                     d.bits, d.group_size, error);
      return FH_OK;
    }
    // Recognised epilogue: out = accumulator + extra (the MoE residual add).
    auto prog = b->programs.find(d.epilogue);
    FH_REQUIRE(prog != b->programs.end());
    fuse_residual = d.accumulator_count == 1 && extras == 1 && prog->second.add_epilogue;
    if (fuse_residual) {
      const fh_tensor &residual = d.inputs[primitive];
      FH_REQUIRE(shape_is(residual, {rows, columns}) && is_float(residual.dtype));
      problem.out = pl.out[0];
      if (try_fast_gather_weighted(b, problem, &pl.in[primitive], error)) return FH_OK;
      if (try_valu_gather_grouped(b, problem, 0, pl.out[0], true, &pl.in[primitive], error)) return FH_OK;
    }
    uint64_t elements = (uint64_t)rows * columns;
    char *acc = b->ensure_workspace(elements * 4);
    if (!acc) return FH_ALLOCATION_FAILED;
    View acc_view = contiguous_view(acc, FH_F32, out);
    if (!try_valu_gather(b, pl.in[0], pl.in[1], pl.in[2], pl.in[3], pl.in[4], &pl.in[5], acc_view, rows,
                         routes, inner, experts, columns, d.bits, d.group_size, error))
      launch_gather_weighted_generic(b->stream, pl.in[0], pl.in[1], pl.in[2], pl.in[3], pl.in[4],
                                     pl.in[5], acc_view, rows, routes, inner, experts, columns,
                                     d.bits, d.group_size, error);
    return run_epilogue(b, pl, primitive, acc, 1);
  }
  // check_gather_quant_projection (ops.rs:1933-1992), once or twice.
  const fh_tensor &idx = d.inputs[primitive - 1];
  FH_REQUIRE(x.rank == 2 && idx.dtype == FH_U32 && idx.rank == 2);
  uint32_t rows = x.shape[0], inner = x.shape[1], k = idx.shape[1];
  FH_REQUIRE(idx.shape[0] == rows);
  fh_status status = check_quant_triple(d.inputs[1], d.inputs[2], d.inputs[3], 3, inner, d.bits,
                                        d.group_size, &columns, &experts);
  if (status != FH_OK) return status;
  if (primitive == 8) {
    uint32_t columns2 = 0, experts2 = 0;
    status = check_quant_triple(d.inputs[4], d.inputs[5], d.inputs[6], 3, inner, d.bits,
                                d.group_size, &columns2, &experts2);
    if (status != FH_OK) return status;
    FH_REQUIRE(columns2 == columns && experts2 == experts);
    FH_REQUIRE(d.epilogue != 0 && d.accumulator_count == 2);
  }
  FH_REQUIRE(shape_is(out, {rows, k, columns}));
  FH_REQUIRE(experts <= 4096);
  if (!execute || rows == 0 || columns == 0 || k == 0) return FH_OK;
  GatherProblem problem{};
  problem.x = pl.in[0];
  problem.packed[0] = pl.in[1];
  problem.scales[0] = pl.in[2];
  problem.biases[0] = pl.in[3];
  if (primitive == 8) {
    problem.packed[1] = pl.in[4];
    problem.scales[1] = pl.in[5];
    problem.biases[1] = pl.in[6];
  }
  problem.indices = pl.in[primitive - 1];
  problem.indices_buffer = d.inputs[primitive - 1].buffer;
  problem.out = pl.out[0];
  problem.rows = rows;
  problem.k = k;
  problem.inner = inner;
  problem.experts = experts;
  problem.columns = columns;
  problem.bits = d.bits;
  problem.group = d.group_size;
  if (!d.epilogue) {
    if (try_fast_gather_projection(b, problem, 1, false, error)) return FH_OK;
    if (try_valu_gather_grouped(b, problem, 0, pl.out[0], false, nullptr, error)) return FH_OK;
    if (try_valu_gather(b, pl.in[0], pl.in[1], pl.in[2], pl.in[3], pl.in[primitive - 1], nullptr, pl.out[0],
                        rows, k, inner, experts, columns, d.bits, d.group_size, error))
      return FH_OK;
    launch_gather_projection_generic(b->stream, pl.in[0], pl.in[1], pl.in[2], pl.in[3],
                                     pl.in[primitive - 1], pl.out[0], rows, inner, experts,
                                     columns, k, d.bits, d.group_size, error);
    return FH_OK;
  }
  auto prog = b->programs.find(d.epilogue);
  FH_REQUIRE(prog != b->programs.end());
  if (primitive == 8 && extras == 0 && prog->second.swiglu_epilogue &&
      try_fast_gather_projection(b, problem, 2, true, error))
    return FH_OK;
  uint32_t accumulators = primitive == 8 ? 2 : 1;
  FH_REQUIRE(d.accumulator_count == accumulators);
  uint64_t elements = (uint64_t)rows * k * columns;
  char *acc = b->ensure_workspace(elements * 4 * accumulators);
  if (!acc) return FH_ALLOCATION_FAILED;
  View acc0 = contiguous_view(acc, FH_F32, out);
  if (!try_valu_gather_grouped(b, problem, 0, acc0, false, nullptr, error) &&
      !try_valu_gather(b, pl.in[0], pl.in[1], pl.in[2], pl.in[3], pl.in[primitive - 1], nullptr, acc0, rows,
                       k, inner, experts, columns, d.bits, d.group_size, error))
    launch_gather_projection_generic(b->stream, pl.in[0], pl.in[1], pl.in[2], pl.in[3],
                                     pl.in[primitive - 1], acc0, rows, inner, experts, columns, k,
                                     d.bits, d.group_size, error);
  if (primitive == 8) {
    View acc1 = contiguous_view(acc + elements * 4, FH_F32, out);
    if (!try_valu_gather_grouped(b, problem, 1, acc1, false, nullptr, error) &&
        !try_valu_gather(b, pl.in[0], pl.in[4], pl.in[5], pl.in[6], pl.in[7], nullptr, acc1, rows, k, inner,
                         experts, columns, d.bits, d.group_size, error))
      launch_gather_projection_generic(b->stream, pl.in[0], pl.in[4], pl.in[5], pl.in[6], pl.in[7],
                                       acc1, rows, inner, experts, columns, k, d.bits, d.group_size,
                                       error);
  }
  return run_epilogue(b, pl, primitive, acc, accumulators);
}

fh_status plan_top_k(fh_backend *b, const Planned &pl, bool execute) {
  const fh_dispatch &d = *pl.d;
  FH_REQUIRE(d.n_inputs == 1 && d.n_outputs == 2);
  const fh_tensor &in = d.inputs[0];
  FH_REQUIRE(is_float(in.dtype) && d.outputs[0].dtype == in.dtype && d.outputs[1].dtype == FH_U32);
  FH_REQUIRE(in.rank >= 1 && in.rank <= 2);
  uint32_t width = in.shape[in.rank - 1];
  FH_REQUIRE(d.k != 0 && d.k <= width && d.k <= 256);
  uint32_t rows = in.rank == 2 ? in.shape[0] : 1;
  for (uint32_t o = 0; o < 2; ++o) {
    FH_REQUIRE(d.outputs[o].rank == in.rank);
    if (in.rank == 2) FH_REQUIRE(d.outputs[o].shape[0] == rows);
    FH_REQUIRE(d.outputs[o].shape[in.rank - 1] == d.k);
  }
  if (!execute) return FH_OK;
  View in_v = pl.in[0], val_v = pl.out[0], idx_v = pl.out[1];
  if (in.rank == 1) {
    for (View *v : {&in_v, &val_v, &idx_v}) {
      v->stride[1] = v->stride[0];
      v->shape[1] = v->shape[0];
      v->stride[0] = 0;
      v->shape[0] = 1;
      v->rank = 2;
    }
  }
  launch_top_k(b->stream, in_v, val_v, idx_v, rows, width, d.k, d.normalize != 0);
  return FH_OK;
}

fh_status plan_argmax(fh_backend *b, const Planned &pl, bool execute) {
  const fh_dispatch &d = *pl.d;
  FH_REQUIRE(d.n_inputs == 1 && d.n_outputs == 1);
  const fh_tensor &in = d.inputs[0], &out = d.outputs[0];
  FH_REQUIRE(is_float(in.dtype) && out.dtype == FH_U32);
  FH_REQUIRE(in.rank >= 1 && in.rank <= 2 && in.shape[in.rank - 1] != 0);
  uint32_t rows = in.rank == 2 ? in.shape[0] : 1;
  FH_REQUIRE(element_count(out) == rows);
  if (!execute) return FH_OK;
  View in_v = pl.in[0];
  if (in.rank == 1) {
    in_v.stride[1] = in_v.stride[0];
    in_v.shape[1] = in_v.shape[0];
    in_v.stride[0] = 0;
    in_v.shape[0] = 1;
    in_v.rank = 2;
  }
  launch_argmax(b->stream, in_v, pl.out[0], rows, in.shape[in.rank - 1]);
  return FH_OK;
}

// check_sample / check_sample_masked (crates/forja-core/src/ops.rs:1546-1592).
fh_status plan_sample(fh_backend *b, const Planned &pl, ErrorSlot *error, bool execute) {
  const fh_dispatch &d = *pl.d;
  const bool masked = d.op == FH_OP_SAMPLE_MASKED;
  FH_REQUIRE(d.n_inputs == (masked ? 3u : 2u) && d.n_outputs == 1);
  const fh_tensor &in = d.inputs[0], &params = d.inputs[1], &out = d.outputs[0];
  FH_REQUIRE(is_float(in.dtype) && out.dtype == FH_U32);
  FH_REQUIRE(params.dtype == FH_U32 && shape_is(params, {5}));
  FH_REQUIRE(in.rank >= 1 && in.rank <= 2 && in.shape[in.rank - 1] != 0);
  const uint32_t rows = in.rank == 2 ? in.shape[0] : 1, width = in.shape[in.rank - 1];
  FH_REQUIRE(element_count(out) == rows);
  if (masked) {
    const fh_tensor &allow = d.inputs[2];
    FH_REQUIRE(allow.dtype == FH_U32 && shape_is(allow, {(width + 31) / 32}) &&
               is_contiguous(allow));
  }
  if (!execute || rows == 0) return FH_OK;
  View in_v = pl.in[0];
  if (in.rank == 1) {
    in_v.stride[1] = in_v.stride[0];
    in_v.shape[1] = in_v.shape[0];
    in_v.stride[0] = 0;
    in_v.shape[0] = 1;
    in_v.rank = 2;
  }
  char *scratch = b->ensure_workspace(sample_scratch_bytes(rows, width));
  if (!scratch) return FH_ALLOCATION_FAILED;
  launch_sample(b->stream, in_v, pl.in[1], masked ? &pl.in[2] : nullptr, pl.out[0], rows, width,
                d.start, scratch, error);
  return FH_OK;
}

fh_status plan_quant_embed(fh_backend *b, const Planned &pl, ErrorSlot *error, bool execute) {
  const fh_dispatch &d = *pl.d;
  FH_REQUIRE(d.n_inputs == 4 && d.n_outputs == 1);
  const fh_tensor &packed = d.inputs[0], &ids = d.inputs[3], &out = d.outputs[0];
  FH_REQUIRE(d.bits == 4 || d.bits == 8);
  FH_REQUIRE(packed.rank == 2 && packed.dtype == FH_U32 && ids.dtype == FH_U32);
  uint32_t vocab = packed.shape[0], packed_width = packed.shape[1];
  uint64_t width64 = (uint64_t)packed_width * (32u / d.bits);
  FH_REQUIRE(width64 <= 0xffffffffull);
  uint32_t width = (uint32_t)width64, columns = 0;
  fh_status status = check_quant_triple(packed, d.inputs[1], d.inputs[2], 2, width, d.bits,
                                        d.group_size, &columns, nullptr);
  if (status != FH_OK) return status;
  FH_REQUIRE(is_float(out.dtype) && out.rank == ids.rank + 1);
  for (uint32_t axis = 0; axis < ids.rank; ++axis) FH_REQUIRE(out.shape[axis] == ids.shape[axis]);
  FH_REQUIRE(out.shape[out.rank - 1] == width);
  if (execute)
    launch_quant_embed(b->stream, pl.in[0], pl.in[1], pl.in[2], pl.in[3], pl.out[0],
                       (uint32_t)element_count(ids), vocab, packed_width, d.bits, d.group_size,
                       error);
  return FH_OK;
}

fh_status plan_matmul(fh_backend *b, const Planned &pl, bool execute) {
  const fh_dispatch &d = *pl.d;
  uint32_t primitive = 2;
  FH_REQUIRE(d.n_outputs == 1 && d.n_inputs == primitive + (d.epilogue ? d.n_extras : 0));
  const fh_tensor &l = d.inputs[0], &r = d.inputs[1], &out = d.outputs[0];
  FH_REQUIRE(is_float(l.dtype) && is_float(r.dtype) && is_float(out.dtype));
  FH_REQUIRE((l.rank == 2 || l.rank == 3) && r.rank == l.rank && out.rank == l.rank);
  uint32_t rank = l.rank;
  uint32_t batches = rank == 3 ? l.shape[0] : 1;
  uint32_t rows = l.shape[rank - 2], inner = l.shape[rank - 1], columns = r.shape[rank - 1];
  FH_REQUIRE(r.shape[rank - 2] == inner && inner != 0);
  if (rank == 3) FH_REQUIRE(r.shape[0] == batches && out.shape[0] == batches);
  FH_REQUIRE(out.shape[rank - 2] == rows && out.shape[rank - 1] == columns);
  if (!execute) return FH_OK;
  if (!d.epilogue) {
    launch_matmul(b->stream, pl.in[0], pl.in[1], pl.out[0], batches, rows, inner, columns);
    return FH_OK;
  }
  uint64_t elements = element_count(out);
  char *acc = b->ensure_workspace(elements * 4);
  if (!acc) return FH_ALLOCATION_FAILED;
  View acc_view = contiguous_view(acc, FH_F32, out);
  launch_matmul(b->stream, pl.in[0], pl.in[1], acc_view, batches, rows, inner, columns);
  return run_epilogue(b, pl, primitive, acc, 1);
}

fh_status plan_rms_norm(fh_backend *b, const Planned &pl, bool execute) {
  const fh_dispatch &d = *pl.d;
  FH_REQUIRE(d.n_inputs == 2 && d.n_outputs == 1);
  const fh_tensor &in = d.inputs[0], &w = d.inputs[1], &out = d.outputs[0];
  FH_REQUIRE(is_float(in.dtype) && is_float(w.dtype) && is_float(out.dtype));
  FH_REQUIRE(in.rank >= 1 && w.rank == 1 && w.shape[0] == in.shape[in.rank - 1] && w.shape[0] != 0);
  FH_REQUIRE(out.rank == in.rank);
  for (uint32_t axis = 0; axis < in.rank; ++axis) FH_REQUIRE(in.shape[axis] == out.shape[axis]);
  FH_REQUIRE(std::isfinite(d.eps) && d.eps >= 0.0f);
  if (execute)
    launch_rms_norm(b->stream, pl.in[0], pl.in[1], pl.out[0],
                    (uint32_t)(element_count(in) / w.shape[0]), w.shape[0], d.eps);
  return FH_OK;
}

fh_status plan_rope(fh_backend *b, const Planned &pl, bool execute) {
  const fh_dispatch &d = *pl.d;
  FH_REQUIRE(d.n_inputs == 2 && d.n_outputs == 1);
  const fh_tensor &in = d.inputs[0], &pos = d.inputs[1], &out = d.outputs[0];
  FH_REQUIRE(is_float(in.dtype) && is_float(out.dtype) && pos.dtype == FH_U32);
  FH_REQUIRE(in.rank == 3 && out.rank == 3 && pos.rank == 1 && pos.shape[0] == in.shape[0]);
  for (uint32_t axis = 0; axis < 3; ++axis) FH_REQUIRE(in.shape[axis] == out.shape[axis]);
  FH_REQUIRE(in.shape[2] % 2 == 0 && std::isfinite(d.theta) && d.theta > 0.0f);
  if (execute)
    launch_rope(b->stream, pl.in[0], pl.in[1], pl.out[0], in.shape[0], in.shape[1], in.shape[2],
                d.theta);
  return FH_OK;
}

// check_paged_copy (ops.rs:1369-1441).
fh_status plan_paged_copy(fh_backend *b, const Planned &pl, ErrorSlot *error, bool execute) {
  const fh_dispatch &d = *pl.d;
  FH_REQUIRE((d.n_inputs == 3 || d.n_inputs == 4) && d.n_outputs == 1);
  bool into = d.direction == 0;
  FH_REQUIRE(d.direction <= 1);
  const fh_tensor &ordinary = into ? d.inputs[0] : d.outputs[0];
  const fh_tensor &pool = into ? d.outputs[0] : d.inputs[0];
  for (uint32_t i = 1; i < d.n_inputs; ++i) FH_REQUIRE(is_contiguous(d.inputs[i]));
  FH_REQUIRE(is_contiguous(pool));
  FH_REQUIRE(is_float(ordinary.dtype) && is_float(pool.dtype));
  FH_REQUIRE(ordinary.rank >= 2 && pool.rank == 3);
  uint64_t elements = 1;
  for (uint32_t axis = 1; axis < ordinary.rank; ++axis) elements *= ordinary.shape[axis];
  uint32_t tokens = ordinary.shape[0];
  FH_REQUIRE(elements <= 0xffffffffull && (uint64_t)tokens * elements <= 0xffffffffull);
  const fh_tensor &table = d.inputs[1], &gens = d.inputs[2];
  FH_REQUIRE(table.dtype == FH_U32 && table.rank == 2 && table.shape[1] == 2);
  FH_REQUIRE(gens.dtype == FH_U32 && shape_is(gens, {pool.shape[0]}));
  if (d.n_inputs == 4) FH_REQUIRE(d.inputs[3].dtype == FH_U32 && shape_is(d.inputs[3], {1}));
  uint64_t capacity = (uint64_t)table.shape[0] * d.page_tokens;
  FH_REQUIRE(d.page_tokens != 0 && pool.shape[1] == d.page_tokens && pool.shape[2] == elements);
  FH_REQUIRE((uint64_t)d.start + tokens <= capacity);
  if (execute) {
    const View &ordinary_v = into ? pl.in[0] : pl.out[0];
    const View &pool_v = into ? pl.out[0] : pl.in[0];
    launch_paged_copy(b->stream, ordinary_v, pool_v, pl.in[1], pl.in[2],
                      d.n_inputs == 4 ? pl.in[3] : null_view(), into, tokens, (uint32_t)elements,
                      d.start, d.page_tokens, pool.shape[0], table.shape[0], error);
  }
  return FH_OK;
}

// check_paged_sdpa (ops.rs:2281-2359) on (q, key pool, value pool, table, generations, activity?).
fh_status check_paged_attention(const fh_tensor &q, const fh_tensor &kp, const fh_tensor &vp,
                                const fh_tensor &table, const fh_tensor &gens,
                                const fh_tensor *activity, const fh_tensor &out, float scale,
                                bool causal, uint32_t q_start, uint32_t key_length,
                                uint32_t page_tokens) {
  FH_REQUIRE(is_contiguous(kp) && is_contiguous(vp) && is_contiguous(table) && is_contiguous(gens));
  if (activity) FH_REQUIRE(is_contiguous(*activity));
  FH_REQUIRE(is_float(q.dtype) && is_float(kp.dtype) && vp.dtype == kp.dtype && is_float(out.dtype));
  FH_REQUIRE(std::isfinite(scale) && page_tokens != 0 && key_length != 0);
  FH_REQUIRE(q.rank == 3 && kp.rank == 4 && vp.rank == 4 && out.rank == 3);
  FH_REQUIRE(table.dtype == FH_U32 && table.rank == 2 && table.shape[1] == 2);
  FH_REQUIRE(gens.dtype == FH_U32 && shape_is(gens, {kp.shape[0]}));
  if (activity) FH_REQUIRE(activity->dtype == FH_U32 && shape_is(*activity, {1}));
  uint64_t capacity = (uint64_t)table.shape[0] * page_tokens;
  FH_REQUIRE(kp.shape[1] == page_tokens && vp.shape[1] == page_tokens);
  FH_REQUIRE(vp.shape[0] == kp.shape[0] && vp.shape[2] == kp.shape[2]);
  FH_REQUIRE(kp.shape[3] == q.shape[2] && kp.shape[2] != 0 && q.shape[0] % kp.shape[2] == 0);
  FH_REQUIRE(q.shape[0] != 0 && key_length <= capacity);
  if (causal) FH_REQUIRE((uint64_t)q_start + q.shape[1] <= key_length);
  FH_REQUIRE(shape_is(out, {q.shape[0], q.shape[1], vp.shape[3]}));
  FH_REQUIRE(q.shape[2] <= 512 && vp.shape[3] <= 256);
  return FH_OK;
}

fh_status plan_paged_sdpa(fh_backend *b, const Planned &pl, ErrorSlot *error, bool execute) {
  const fh_dispatch &d = *pl.d;
  FH_REQUIRE((d.n_inputs == 5 || d.n_inputs == 6) && d.n_outputs == 1);
  const fh_tensor *activity = d.n_inputs == 6 ? &d.inputs[5] : nullptr;
  fh_status status =
      check_paged_attention(d.inputs[0], d.inputs[1], d.inputs[2], d.inputs[3], d.inputs[4],
                            activity, d.outputs[0], d.scale, d.causal != 0, d.q_start,
                            d.key_length, d.page_tokens);
  if (status != FH_OK) return status;
  if (!execute) return FH_OK;
  const fh_tensor &q = d.inputs[0], &kp = d.inputs[1], &vp = d.inputs[2];
  LaneAttention lane{pl.in[0], pl.in[1], pl.in[2], pl.in[3], pl.in[4],
                     activity ? pl.in[5] : null_view(), pl.out[0], q.shape[0], q.shape[1],
                     kp.shape[2], q.shape[2], vp.shape[3], d.key_length, d.q_start, d.scale,
                     d.causal != 0, d.page_tokens, kp.shape[0], d.inputs[3].shape[0]};
  if (try_fast_lane_attention(b, lane, error)) return FH_OK;
  launch_paged_sdpa_generic(b->stream, lane.q, lane.key_pool, lane.value_pool, lane.table,
                            lane.generations, lane.activity, lane.out, lane.query_heads,
                            lane.query_length, lane.kv_heads, lane.width, lane.value_width,
                            lane.key_length, lane.query_start, lane.scale, lane.causal,
                            lane.page_tokens, lane.physical_pages, lane.logical_pages, error);
  return FH_OK;
}

// check_paged_append (ops.rs:2236-2278): inputs (q, k_new, v_new, table, generations, activity?),
// outputs (attention, key pool, value pool).
fh_status plan_paged_append(fh_backend *b, const Planned &pl, ErrorSlot *error, bool execute) {
  const fh_dispatch &d = *pl.d;
  FH_REQUIRE((d.n_inputs == 5 || d.n_inputs == 6) && d.n_outputs == 3);
  FH_REQUIRE(d.q_start != 0xffffffffu);
  const fh_tensor *activity = d.n_inputs == 6 ? &d.inputs[5] : nullptr;
  const fh_tensor &q = d.inputs[0], &kp = d.outputs[1], &vp = d.outputs[2];
  fh_status status = check_paged_attention(q, kp, vp, d.inputs[3], d.inputs[4], activity,
                                           d.outputs[0], d.scale, true, d.q_start, d.q_start + 1,
                                           d.page_tokens);
  if (status != FH_OK) return status;
  FH_REQUIRE(kp.shape[3] == vp.shape[3] && q.shape[1] == 1);
  FH_REQUIRE(kp.buffer != vp.buffer);
  for (uint32_t index : {1u, 2u}) {
    const fh_tensor &pool = d.outputs[index];
    FH_REQUIRE(d.inputs[index].dtype == q.dtype);
    FH_REQUIRE(shape_is(d.inputs[index], {1, pool.shape[2], pool.shape[3]}));
  }
  if (!execute) return FH_OK;
  // Store both planes, then attend through them (lib.rs:262-306).
  View act = activity ? pl.in[5] : null_view();
  for (uint32_t index : {1u, 2u}) {
    const fh_tensor &pool = d.outputs[index];
    launch_paged_copy(b->stream, pl.in[index], pl.out[index], pl.in[3], pl.in[4], act, true, 1,
                      pool.shape[2] * pool.shape[3], d.q_start, d.page_tokens, pool.shape[0],
                      d.inputs[3].shape[0], error);
  }
  LaneAttention lane{pl.in[0], pl.out[1], pl.out[2], pl.in[3], pl.in[4], act, pl.out[0],
                     q.shape[0], 1, kp.shape[2], q.shape[2], vp.shape[3], d.q_start + 1,
                     d.q_start, d.scale, true, d.page_tokens, kp.shape[0], d.inputs[3].shape[0]};
  if (try_fast_lane_attention(b, lane, error)) return FH_OK;
  launch_paged_sdpa_generic(b->stream, lane.q, lane.key_pool, lane.value_pool, lane.table,
                            lane.generations, lane.activity, lane.out, lane.query_heads, 1,
                            lane.kv_heads, lane.width, lane.value_width, lane.key_length,
                            lane.query_start, lane.scale, true, lane.page_tokens,
                            lane.physical_pages, lane.logical_pages, error);
  return FH_OK;
}

fh_status plan_ragged(fh_backend *b, const Planned &pl, ErrorSlot *error, bool execute) {
  const fh_dispatch &d = *pl.d;
  FH_REQUIRE((d.n_inputs == 7 || d.n_inputs == 8) && d.n_outputs == 3);
  const fh_tensor &q = d.inputs[0], &kn = d.inputs[1], &vn = d.inputs[2], &tables = d.inputs[3],
                  &gens = d.inputs[4], &cu = d.inputs[5], &starts = d.inputs[6];
  const fh_tensor &out = d.outputs[0], &kp = d.outputs[1], &vp = d.outputs[2];
  for (uint32_t i = 3; i < d.n_inputs; ++i)
    FH_REQUIRE(is_contiguous(d.inputs[i]) && d.inputs[i].dtype == FH_U32);
  FH_REQUIRE(is_contiguous(kp) && is_contiguous(vp) && kp.buffer != vp.buffer);
  FH_REQUIRE(is_float(q.dtype) && kn.dtype == q.dtype && vn.dtype == q.dtype);
  FH_REQUIRE(is_float(kp.dtype) && vp.dtype == kp.dtype && is_float(out.dtype));
  FH_REQUIRE(q.rank == 3 && kn.rank == 3 && vn.rank == 3 && out.rank == 3);
  FH_REQUIRE(kp.rank == 4 && vp.rank == 4 && tables.rank == 3 && tables.shape[2] == 2);
  uint32_t tokens = q.shape[0], lanes = tables.shape[0];
  FH_REQUIRE(lanes != 0 && shape_is(cu, {lanes + 1}) && shape_is(starts, {lanes}));
  if (d.n_inputs == 8) FH_REQUIRE(shape_is(d.inputs[7], {lanes}));
  FH_REQUIRE(shape_is(gens, {kp.shape[0]}));
  FH_REQUIRE(std::isfinite(d.scale) && d.page_tokens != 0 && d.k <= 1);
  FH_REQUIRE(kp.shape[1] == d.page_tokens && vp.shape[1] == d.page_tokens);
  FH_REQUIRE(vp.shape[0] == kp.shape[0] && vp.shape[2] == kp.shape[2]);
  FH_REQUIRE(kp.shape[2] != 0 && q.shape[1] % kp.shape[2] == 0 && q.shape[1] != 0);
  FH_REQUIRE(kp.shape[3] == q.shape[2]);
  FH_REQUIRE(shape_is(kn, {tokens, kp.shape[2], kp.shape[3]}));
  FH_REQUIRE(shape_is(vn, {tokens, vp.shape[2], vp.shape[3]}));
  FH_REQUIRE(shape_is(out, {tokens, q.shape[1], vp.shape[3]}));
  FH_REQUIRE(q.shape[2] <= 512 && vp.shape[3] <= 256);
  if (!execute || tokens == 0) return FH_OK;
  RaggedAttention problem{};
  problem.q = pl.in[0];
  problem.k_new = pl.in[1];
  problem.v_new = pl.in[2];
  problem.tables = pl.in[3];
  problem.generations = pl.in[4];
  problem.cu_seqlens = pl.in[5];
  problem.q_starts = pl.in[6];
  problem.activity = d.n_inputs == 8 ? pl.in[7] : null_view();
  problem.out = pl.out[0];
  problem.key_pool = pl.out[1];
  problem.value_pool = pl.out[2];
  problem.tokens = tokens;
  problem.lanes = lanes;
  problem.query_heads = q.shape[1];
  problem.kv_heads = kp.shape[2];
  problem.width = q.shape[2];
  problem.value_width = vp.shape[3];
  problem.page_tokens = d.page_tokens;
  problem.physical_pages = kp.shape[0];
  problem.table_pages = tables.shape[1];
  problem.scale = d.scale;
  problem.metadata_buffers[0] = d.inputs[5].buffer;
  problem.metadata_buffers[1] = d.inputs[6].buffer;
  problem.metadata_buffers[2] = d.n_inputs == 8 ? d.inputs[7].buffer : 0;
  problem.metadata_buffers[3] = d.inputs[3].buffer;
  problem.metadata_buffers[4] = d.inputs[4].buffer;
  problem.one_row_per_lane = d.k == 1;
  if (!run_ragged_attention(b, problem, error)) return FH_ALLOCATION_FAILED;
  return FH_OK;
}

fh_status plan_route_pack(fh_backend *b, const Planned &pl, ErrorSlot *error, bool execute) {
  const fh_dispatch &d = *pl.d;
  FH_REQUIRE(d.n_inputs == 1 && d.n_outputs == 4);
  const fh_tensor &idx = d.inputs[0];
  FH_REQUIRE(idx.dtype == FH_U32 && idx.rank == 2);
  for (uint32_t o = 0; o < 4; ++o)
    FH_REQUIRE(d.outputs[o].dtype == FH_U32 && is_contiguous(d.outputs[o]));
  uint32_t experts = d.outputs[0].shape[0];
  FH_REQUIRE(d.outputs[0].rank == 1 && experts != 0);
  if (experts > 512) return FH_UNSUPPORTED_OPERATION;  // per-wave counts of all experts live in LDS
  FH_REQUIRE(shape_is(d.outputs[1], {experts + 1}));
  uint64_t routes = (uint64_t)idx.shape[0] * idx.shape[1];
  FH_REQUIRE(routes <= (1u << 24) && shape_is(d.outputs[2], {(uint32_t)routes}));
  FH_REQUIRE(d.outputs[3].rank == 2 && d.outputs[3].shape[1] == 3 && d.k != 0);
  uint32_t max_blocks = d.outputs[3].shape[0];
  FH_REQUIRE(max_blocks >= experts + routes / d.k);
  if (!execute) return FH_OK;
  char *ws = b->ensure_workspace(256);
  if (!ws) return FH_ALLOCATION_FAILED;
  auto ptr = [](const View &v) { return (uint32_t *)v.base + v.offset; };
  launch_route_pack(b->stream, pl.in[0], idx.shape[0], idx.shape[1], experts, d.k, ptr(pl.out[0]),
                    ptr(pl.out[1]), ptr(pl.out[2]), ptr(pl.out[3]), max_blocks, (uint32_t *)ws,
                    error);
  return FH_OK;
}

fh_status plan_fill(fh_backend *b, const Planned &pl, bool execute) {
  const fh_dispatch &d = *pl.d;
  FH_REQUIRE(d.n_inputs == 0 && d.n_outputs == 1 && d.k <= 2);
  const fh_tensor &out = d.outputs[0];
  FH_REQUIRE(is_contiguous(out));
  if (d.k == 0)
    FH_REQUIRE(out.dtype == FH_U32);
  else
    FH_REQUIRE(is_float(out.dtype));
  if (execute) {
    uint64_t seed = (uint64_t)d.q_start | ((uint64_t)d.key_length << 32);
    launch_fill_seeded(b->stream, pl.out[0], element_count(out), d.k, seed, d.start, d.direction,
                       d.scale, d.eps);
  }
  return FH_OK;
}

uint32_t kernel_class_of(uint32_t op) {
  switch (op) {
  case FH_OP_QUANT_MATMUL: return FH_KC_QMM;
  case FH_OP_GATHER_QUANT_MATMUL: return FH_KC_MOE;
  case FH_OP_PAGED_SDPA:
  case FH_OP_PAGED_SDPA_APPEND:
  case FH_OP_PAGED_ATTENTION_RAGGED: return FH_KC_ATTENTION;
  default: return FH_KC_OTHER;
  }
}

// Validates one dispatch and, when `execute`, enqueues it.
fh_status process(fh_backend *b, const fh_dispatch &d, ErrorSlot *error, bool execute) {
  FH_REQUIRE(d.n_inputs <= FH_MAX_INPUTS && d.n_outputs <= FH_MAX_OUTPUTS && d.n_outputs >= 1);
  Planned pl;
  pl.d = &d;
  for (uint32_t i = 0; i < d.n_inputs; ++i) {
    fh_status status = make_view(b, d.inputs[i], false, &pl.in[i]);
    if (status != FH_OK) return status;
  }
  for (uint32_t i = 0; i < d.n_outputs; ++i) {
    fh_status status = make_view(b, d.outputs[i], true, &pl.out[i]);
    if (status != FH_OK) return status;
  }
  // Outputs must not alias inputs or each other (check_common, ops.rs:1300-1344).
  for (uint32_t o = 0; o < d.n_outputs; ++o) {
    for (uint32_t i = 0; i < d.n_inputs; ++i) FH_REQUIRE(!may_overlap(d.outputs[o], d.inputs[i]));
    for (uint32_t other = o + 1; other < d.n_outputs; ++other)
      FH_REQUIRE(!may_overlap(d.outputs[o], d.outputs[other]));
  }
  switch (d.op) {
  case FH_OP_PROGRAM: return plan_program(b, pl, execute);
  case FH_OP_COPY: return plan_copy(b, pl, execute);
  case FH_OP_PAGED_COPY: return plan_paged_copy(b, pl, error, execute);
  case FH_OP_RMS_NORM: return plan_rms_norm(b, pl, execute);
  case FH_OP_ARGMAX: return plan_argmax(b, pl, execute);
  case FH_OP_SAMPLE:
  case FH_OP_SAMPLE_MASKED: return plan_sample(b, pl, error, execute);
  case FH_OP_TOP_K: return plan_top_k(b, pl, execute);
  case FH_OP_ROPE: return plan_rope(b, pl, execute);
  case FH_OP_QUANT_EMBED: return plan_quant_embed(b, pl, error, execute);
  case FH_OP_MATMUL: return plan_matmul(b, pl, execute);
  case FH_OP_QUANT_MATMUL: return plan_quant_matmul(b, pl, error, execute);
  case FH_OP_GATHER_QUANT_MATMUL: return plan_gather(b, pl, error, execute);
  case FH_OP_PAGED_SDPA_APPEND: return plan_paged_append(b, pl, error, execute);
  case FH_OP_PAGED_SDPA: return plan_paged_sdpa(b, pl, error, execute);
  case FH_OP_PAGED_ATTENTION_RAGGED: return plan_ragged(b, pl, error, execute);
  case FH_OP_ROUTE_PACK: return plan_route_pack(b, pl, error, execute);
  case FH_OP_FILL_SEEDED: return plan_fill(b, pl, execute);
  default: return FH_UNSUPPORTED_OPERATION;
  }
}

// ---------------------------------------------------------------- a normalisation after a sum
//
// Every decoder layer ends with the MoE weighted sum (+ residual) into the hidden rows and the
// next layer begins with the RMS normalisation of exactly those rows
// (engines/qwen3-coder/src/lib.rs records them back to back).  When `next` is that normalisation
// of what `d` produces, the kernel that forms the rows can write the normalised rows too: same
// values, one launch less.  Nothing is assumed: `next` is validated as the dispatch it is, reads
// the produced tensor element for element, and writes nothing that `d` still reads.
bool find_norm_tail(fh_backend *b, const fh_dispatch &d, const fh_dispatch &next, NormTail *tail) {
  if (d.op != FH_OP_GATHER_QUANT_MATMUL || next.op != FH_OP_PROGRAM || b->static_mode) return false;
  if (d.n_outputs != 1 || next.n_inputs != 2 || next.n_outputs != 1) return false;
  auto program = b->programs.find(next.program);
  if (program == b->programs.end() || program->second.fast.kind != kProgramRmsNorm) return false;
  const fh_tensor &made = d.outputs[0], &read = next.inputs[0];
  if (made.buffer != read.buffer || made.offset != read.offset || made.rank != 2 || read.rank != 2 ||
      made.dtype != read.dtype)
    return false;
  for (uint32_t axis = 0; axis < 2; ++axis)
    if (made.shape[axis] != read.shape[axis] || made.stride[axis] != read.stride[axis]) return false;
  // rows of the sum are still being formed while normalised rows are written, and the weights
  // of the normalisation are read while rows of the sum are written
  for (uint32_t i = 0; i < d.n_inputs && i < FH_MAX_INPUTS; ++i)
    if (may_overlap(next.outputs[0], d.inputs[i])) return false;
  if (may_overlap(next.outputs[0], made) || may_overlap(next.inputs[1], made)) return false;
  if (process(b, next, nullptr, false) != FH_OK) return false;
  View in[2], out, produced;
  if (make_view(b, next.inputs[0], false, &in[0]) != FH_OK ||
      make_view(b, next.inputs[1], false, &in[1]) != FH_OK ||
      make_view(b, next.outputs[0], true, &out) != FH_OK || make_view(b, made, true, &produced) != FH_OK)
    return false;
  ProgramArgs args;
  if (bind_program(b, program->second, next.inputs, 2, in, next.outputs, 1, &out, next.outputs[0].shape,
                   next.outputs[0].rank, &args) != FH_OK)
    return false;
  return norm_tail_of(program->second.fast, args, produced, tail);
}

// ---------------------------------------------------------------- fusion of per-lane attention
//
// The engines record a decode batch lane by lane (engines/qwen3-coder/src/lib.rs:917-935): for
// every lane one Op::PagedSdpaAppend on narrowed rows of the packed q/k/v activations, with the
// lane's own block-table allocation and a freshly allocated output row
// (crates/forja-sdk/src/paged.rs:525-528), followed by the Op::Copy of that row into the packed
// `attended` activation.  Executed one by one that is hundreds of tiny launches per layer.  A run
// of such dispatches is recognised here and executed as: one gather of the lanes' metadata (kept
// for the other layers of the submission), one ragged attention launch into scratch rows, one
// scatter of the rows to the places the dispatches named.  The result is what serial execution
// gives as long as no member reads what another member writes, which the checks below establish
// from the tensors alone (allocation identities and element spans); a run that fails any check
// is executed serially.  One thing is taken from the host rather than proved: a lane's appended
// slot lies outside every other lane's attended range (pages are copy-on-write,
// crates/forja-host/src/lib.rs:5408-5470), which also makes the key/value writes of different
// members independent.

// One lane's share of a run, whichever way it was recorded.
struct LaneMember {
  fh_tensor q, k_new, v_new;  // [heads, 1, D]; [1, kv heads, D] twice
  fh_tensor table, generations, activity, out, key_pool, value_pool;  // pools as [P, pt, Hkv, D]
  bool has_activity = false;
  bool has_copy = false;      // an Op::Copy of the output row follows
  fh_tensor copy_target{};
  uint32_t q_start = 0, page_tokens = 0;
  uint32_t tokens = 1;        // query rows (more than one: a prefill chunk, see chunk_member_at)
  float scale = 0.0f;
  uint32_t dispatches = 0;    // dispatches of the member, the copy included
  uint32_t attention_at = 0;  // which of them is the attention (its failures are recorded there)
};

struct LaneRun {
  std::vector<LaneMember> members;
  uint32_t dispatches = 0;       // examined (and, when fused, replaced)
  int64_t delta[3] = {0, 0, 0};  // element distance between consecutive members' q, k_new, v_new
};

bool same_layout(const fh_tensor &a, const fh_tensor &b) {
  if (a.dtype != b.dtype || a.rank != b.rank) return false;
  for (uint32_t axis = 0; axis < a.rank; ++axis)
    if (a.shape[axis] != b.shape[axis] || a.stride[axis] != b.stride[axis]) return false;
  return true;
}

bool same_tensor(const fh_tensor &a, const fh_tensor &b) {
  return a.buffer == b.buffer && a.offset == b.offset && same_layout(a, b);
}

// The [heads, 1, width] attention output as one dense row of heads * width elements.
bool dense_head_rows(const fh_tensor &out) {
  return out.rank == 3 && out.shape[1] == 1 && out.stride[2] == 1 && out.stride[0] == out.shape[2];
}

// `copy` moves exactly the row `out`, unconverted, into a dense destination.
bool copies_attended_row(const fh_tensor &row, const fh_dispatch &copy) {
  if (copy.op != FH_OP_COPY || copy.n_inputs != 1 || copy.n_outputs != 1) return false;
  const fh_tensor &in = copy.inputs[0], &out = copy.outputs[0];
  return in.buffer == row.buffer && in.offset == row.offset && in.dtype == row.dtype &&
         out.dtype == row.dtype && is_contiguous(in) && is_contiguous(out) &&
         element_count(in) == (uint64_t)row.shape[0] * row.shape[2] &&
         element_count(out) == element_count(in);
}

// A [1, ...] row of `heads * width` contiguous elements as the tensor [1, heads, width].
bool as_head_rows(const fh_tensor &row, uint32_t heads, uint32_t width, fh_tensor *out) {
  if (row.rank < 2 || row.shape[0] != 1 || !is_contiguous(row)) return false;
  if (element_count(row) != (uint64_t)heads * width) return false;
  *out = row;
  out->rank = 3;
  out->shape[0] = 1;
  out->shape[1] = heads;
  out->shape[2] = width;
  out->stride[0] = (uint64_t)heads * width;
  out->stride[1] = width;
  out->stride[2] = 1;
  return true;
}

// Reads the lane recorded at `at` in either idiom: Op::PagedSdpaAppend
// (engines/qwen3-coder/src/lib.rs:917-935), or two Op::PagedCopy{IntoPages} of the lane's key and
// value row followed by Op::PagedSdpa over one query row
// (engines/qwen38/src/attention/batch.rs:37-53); each optionally followed by the row's Op::Copy.
// Every dispatch has passed its own validation before this is called.
bool lane_member_at(const fh_dispatch *d, uint32_t count, uint32_t at, LaneMember *m) {
  const fh_dispatch &first = d[at];
  *m = LaneMember{};
  if (first.op == FH_OP_PAGED_SDPA_APPEND) {
    if (first.n_outputs != 3 || (first.n_inputs != 5 && first.n_inputs != 6)) return false;
    m->q = first.inputs[0];
    m->k_new = first.inputs[1];
    m->v_new = first.inputs[2];
    m->table = first.inputs[3];
    m->generations = first.inputs[4];
    m->has_activity = first.n_inputs == 6;
    if (m->has_activity) m->activity = first.inputs[5];
    m->out = first.outputs[0];
    m->key_pool = first.outputs[1];
    m->value_pool = first.outputs[2];
    m->q_start = first.q_start;
    m->page_tokens = first.page_tokens;
    m->scale = first.scale;
    m->dispatches = 1;
    m->attention_at = 0;
  } else if (first.op == FH_OP_PAGED_COPY) {
    if (at + 2 >= count) return false;
    const fh_dispatch &second = d[at + 1], &attention = d[at + 2];
    if (second.op != FH_OP_PAGED_COPY || attention.op != FH_OP_PAGED_SDPA) return false;
    if (first.direction != 0 || second.direction != 0) return false;
    if (first.n_inputs != second.n_inputs || attention.n_inputs != first.n_inputs + 2) return false;
    if (attention.n_outputs != 1 || attention.inputs[0].shape[1] != 1) return false;
    const fh_tensor &kp = attention.inputs[1], &vp = attention.inputs[2];
    // both copies write the pools the attention reads, one row at its query position
    if (first.outputs[0].buffer != kp.buffer || first.outputs[0].offset != kp.offset ||
        first.outputs[0].dtype != kp.dtype || second.outputs[0].buffer != vp.buffer ||
        second.outputs[0].offset != vp.offset || second.outputs[0].dtype != vp.dtype)
      return false;
    if (first.start != attention.q_start || second.start != attention.q_start ||
        attention.key_length != attention.q_start + 1 || first.page_tokens != attention.page_tokens ||
        second.page_tokens != attention.page_tokens)
      return false;
    for (const fh_dispatch *copy : {&first, &second}) {
      if (!same_tensor(copy->inputs[1], attention.inputs[3]) ||
          !same_tensor(copy->inputs[2], attention.inputs[4]))
        return false;
      if (copy->n_inputs == 4 && !same_tensor(copy->inputs[3], attention.inputs[5])) return false;
    }
    if (!as_head_rows(first.inputs[0], kp.shape[2], kp.shape[3], &m->k_new) ||
        !as_head_rows(second.inputs[0], vp.shape[2], vp.shape[3], &m->v_new))
      return false;
    m->q = attention.inputs[0];
    m->table = attention.inputs[3];
    m->generations = attention.inputs[4];
    m->has_activity = attention.n_inputs == 6;
    if (m->has_activity) m->activity = attention.inputs[5];
    m->out = attention.outputs[0];
    m->key_pool = kp;
    m->value_pool = vp;
    m->q_start = attention.q_start;
    m->page_tokens = attention.page_tokens;
    m->scale = attention.scale;
    m->dispatches = 3;
    m->attention_at = 2;
  } else {
    return false;
  }
  if (m->k_new.dtype != m->q.dtype || m->v_new.dtype != m->q.dtype) return false;
  if (!dense_head_rows(m->out) || !is_contiguous(m->table)) return false;
  if (m->has_activity && element_count(m->activity) != 1) return false;
  if (at + m->dispatches < count && copies_attended_row(m->out, d[at + m->dispatches])) {
    m->has_copy = true;
    m->copy_target = d[at + m->dispatches].outputs[0];
    m->dispatches += 1;
  }
  return true;
}

bool same_lane_shape(const LaneMember &a, const LaneMember &b) {
  if (a.dispatches != b.dispatches || a.attention_at != b.attention_at ||
      a.has_activity != b.has_activity || a.has_copy != b.has_copy)
    return false;
  if (memcmp(&a.scale, &b.scale, sizeof(float)) != 0 || a.page_tokens != b.page_tokens) return false;
  const fh_tensor *left[3] = {&a.q, &a.k_new, &a.v_new}, *right[3] = {&b.q, &b.k_new, &b.v_new};
  for (uint32_t i = 0; i < 3; ++i)
    if (left[i]->buffer != right[i]->buffer || !same_layout(*left[i], *right[i])) return false;
  if (!same_layout(a.table, b.table) || !same_tensor(a.generations, b.generations)) return false;
  if (a.has_activity && !same_layout(a.activity, b.activity)) return false;
  if (a.has_copy && !same_layout(a.copy_target, b.copy_target)) return false;
  return same_layout(a.out, b.out) && same_tensor(a.key_pool, b.key_pool) &&
         same_tensor(a.value_pool, b.value_pool);
}

// Longest fusable run of per-lane attention starting at `first`; false when there is none of at
// least two lanes.  `run->dispatches` then still says how many dispatches were examined, so that
// the caller does not examine the tail of a refused run again.
bool find_lane_run(const fh_dispatch *d, uint32_t count, uint32_t first, LaneRun *run) {
  *run = LaneRun{};
  LaneMember member;
  if (!lane_member_at(d, count, first, &member)) return false;
  run->members.push_back(member);
  run->dispatches = member.dispatches;
  for (;;) {
    const uint32_t at = first + run->dispatches;
    if (at >= count || !lane_member_at(d, count, at, &member)) break;
    const LaneMember &head = run->members[0];
    if (!same_lane_shape(head, member)) break;
    const fh_tensor *mine[3] = {&member.q, &member.k_new, &member.v_new};
    const fh_tensor *heads[3] = {&head.q, &head.k_new, &head.v_new};
    bool regular = true;
    const int64_t index = (int64_t)run->members.size();
    for (uint32_t i = 0; i < 3; ++i) {
      int64_t distance = (int64_t)mine[i]->offset - (int64_t)heads[i]->offset;
      if (index == 1) {
        if (distance <= 0) regular = false;
        run->delta[i] = distance;
      } else if (distance != run->delta[i] * index) {
        regular = false;
      }
    }
    if (!regular) break;
    run->members.push_back(member);
    run->dispatches += member.dispatches;
  }
  if (run->members.size() < 2) return false;
  // Nothing a member writes may be something another member reads or writes.
  const LaneMember &head = run->members[0];
  std::unordered_set<uint64_t> read;
  for (const fh_tensor *t : {&head.q, &head.k_new, &head.v_new, &head.generations, &head.key_pool,
                             &head.value_pool})
    read.insert(t->buffer);
  struct Span {
    uint64_t buffer, lo, hi;
  };
  std::vector<Span> written;
  written.reserve(run->members.size() * 2);
  for (const LaneMember &m : run->members) {
    read.insert(m.table.buffer);
    if (m.has_activity) read.insert(m.activity.buffer);
    const uint64_t row = (uint64_t)m.out.shape[0] * m.out.shape[2];
    written.push_back({m.out.buffer, m.out.offset, m.out.offset + row});
    if (m.has_copy)
      written.push_back({m.copy_target.buffer, m.copy_target.offset, m.copy_target.offset + row});
  }
  for (const Span &span : written)
    if (read.count(span.buffer)) return false;
  // Two members on one table would append to the same slot: order matters, so no fusion.
  {
    std::vector<std::pair<uint64_t, uint64_t>> tables;
    tables.reserve(run->members.size());
    for (const LaneMember &m : run->members) tables.push_back({m.table.buffer, m.table.offset});
    std::sort(tables.begin(), tables.end());
    if (std::adjacent_find(tables.begin(), tables.end()) != tables.end()) return false;
  }
  std::sort(written.begin(), written.end(), [](const Span &a, const Span &b) {
    return a.buffer != b.buffer ? a.buffer < b.buffer : a.lo < b.lo;
  });
  for (size_t i = 1; i < written.size(); ++i)
    if (written[i].buffer == written[i - 1].buffer && written[i].lo < written[i - 1].hi) return false;
  return true;
}

// Executes the run found by find_lane_run.  `errors` is the record of the run's first dispatch;
// member i's records start at errors[i * dispatches per member].
// `*executed` is false when the lanes' tables overlap in a way that makes the order of the
// dispatches matter: nothing of the run has been executed then and the caller runs it one by one.
fh_status run_lane_group(fh_backend *b, const LaneRun &run, ErrorSlot *errors, bool *executed) {
  *executed = true;
  const LaneMember &head = run.members[0];
  const fh_tensor &q0 = head.q, &out0 = head.out, &kp = head.key_pool, &vp = head.value_pool;
  const uint32_t lanes = (uint32_t)run.members.size(), heads = q0.shape[0];
  const uint32_t table_pages = head.table.shape[0], table_words = table_pages * 2;
  const uint64_t row_bytes = (uint64_t)heads * out0.shape[2] * dtype_size(out0.dtype);
  FH_REQUIRE(row_bytes < (1ull << 31));
  const uint64_t metadata_words = (uint64_t)lanes * table_words + 3ull * lanes + 2;
  const uint64_t rows_at = (metadata_words * 4 + 255) / 256 * 256;
  char *scratch = b->ensure_lane_scratch(rows_at + lanes * row_bytes);
  if (!scratch) return FH_ALLOCATION_FAILED;
  uint32_t *tables = (uint32_t *)scratch;
  uint32_t *activity = tables + (uint64_t)lanes * table_words;
  uint32_t *starts = activity + lanes;
  uint32_t *cu = starts + lanes;
  char *rows = scratch + rows_at;

  // What the gathered metadata depends on; equal keys mean the gather of an earlier layer holds.
  std::vector<uint64_t> key;
  key.reserve(5ull * lanes + 2);
  key.push_back(lanes);
  key.push_back(table_words);
  for (const LaneMember &m : run.members) {
    key.push_back(m.table.buffer);
    key.push_back(m.table.offset);
    key.push_back(m.has_activity ? m.activity.buffer : 0);
    key.push_back(m.has_activity ? m.activity.offset : 0);
    key.push_back(m.q_start);
  }
  fh_status status;
  if (!(b->lane_metadata_valid && key == b->lane_metadata_key)) {
    b->lane_metadata_valid = false;
    b->attention_plan_valid = false;  // the plan was built from the metadata replaced here
    b->lane_metadata_watch.clear();
    for (uint32_t base = 0; base < lanes; base += kLaneChunk) {
      uint32_t chunk = std::min<uint32_t>(kLaneChunk, lanes - base);
      LaneSources sources{};
      for (uint32_t local = 0; local < chunk; ++local) {
        const LaneMember &m = run.members[base + local];
        View table, flag;
        if ((status = make_view(b, m.table, false, &table)) != FH_OK) return status;
        sources.table[local] = (const uint32_t *)table.base + table.offset;
        b->lane_metadata_watch.insert(m.table.buffer);
        if (m.has_activity) {
          if ((status = make_view(b, m.activity, false, &flag)) != FH_OK) return status;
          sources.activity[local] = (const uint32_t *)flag.base + flag.offset;
          b->lane_metadata_watch.insert(m.activity.buffer);
        }
        sources.start[local] = m.q_start;
      }
      launch_gather_lane_metadata(b->stream, sources, base, chunk, lanes, table_words, tables,
                                  activity, starts, cu);
    }
    // The one thing the tensors cannot show: an append into a slot another lane attends.  Checked
    // on the gathered tables, once per set of tables (not per layer); the verdict is needed here,
    // so the stream is waited for.
    uint32_t *flag = cu + lanes + 1;
    b->lane_conflict = true;
    if (launch_lane_conflict_check(b->stream, tables, activity, starts, lanes, table_pages,
                                   head.page_tokens, flag)) {
      if (hipMemcpyAsync(b->host_flag, flag, sizeof(uint32_t), hipMemcpyDeviceToHost, b->stream) != hipSuccess ||
          hipStreamSynchronize(b->stream) != hipSuccess)
        return FH_DEVICE_EXECUTION_FAILED;
      b->lane_conflict = *b->host_flag != 0;
    }
    b->lane_metadata_key = std::move(key);
    b->lane_metadata_valid = true;
  }
  if (b->lane_conflict) {
    *executed = false;
    return FH_OK;
  }

  auto device_view = [](char *base, uint32_t dtype, std::initializer_list<uint32_t> shape) {
    View v{};
    v.base = base;
    v.dtype = dtype;
    v.rank = (uint32_t)shape.size();
    for (uint32_t axis = 0; axis < FH_MAX_RANK; ++axis) {
      v.shape[axis] = 1;
      v.stride[axis] = 0;
    }
    uint32_t axis = 0;
    for (uint32_t extent : shape) v.shape[axis++] = extent;
    uint64_t stride = 1;
    for (int at = (int)v.rank - 1; at >= 0; --at) {
      v.stride[at] = stride;
      stride *= v.shape[at];
    }
    return v;
  };
  RaggedAttention problem{};
  // q [heads, 1, D] per member -> [lanes, heads, D]; k_new / v_new [1, Hkv, D] -> [lanes, Hkv, D].
  if ((status = make_view(b, q0, false, &problem.q)) != FH_OK) return status;
  problem.q.shape[0] = lanes;
  problem.q.shape[1] = heads;
  problem.q.stride[0] = (uint64_t)run.delta[0];
  problem.q.stride[1] = q0.stride[0];
  View *appended[2] = {&problem.k_new, &problem.v_new};
  const fh_tensor *appended_from[2] = {&head.k_new, &head.v_new};
  for (uint32_t i = 0; i < 2; ++i) {
    if ((status = make_view(b, *appended_from[i], false, appended[i])) != FH_OK) return status;
    appended[i]->shape[0] = lanes;
    appended[i]->stride[0] = (uint64_t)run.delta[1 + i];
  }
  if ((status = make_view(b, head.generations, false, &problem.generations)) != FH_OK) return status;
  if ((status = make_view(b, kp, true, &problem.key_pool)) != FH_OK) return status;
  if ((status = make_view(b, vp, true, &problem.value_pool)) != FH_OK) return status;
  problem.tables = device_view((char *)tables, FH_U32, {lanes, table_pages, 2});
  problem.activity = device_view((char *)activity, FH_U32, {lanes});
  problem.q_starts = device_view((char *)starts, FH_U32, {lanes});
  problem.cu_seqlens = device_view((char *)cu, FH_U32, {lanes + 1});
  problem.out = device_view(rows, out0.dtype, {lanes, heads, out0.shape[2]});
  problem.tokens = lanes;
  problem.lanes = lanes;
  problem.query_heads = heads;
  problem.kv_heads = kp.shape[2];
  problem.width = q0.shape[2];
  problem.value_width = vp.shape[3];
  problem.page_tokens = head.page_tokens;
  problem.physical_pages = kp.shape[0];
  problem.table_pages = table_pages;
  problem.scale = head.scale;
  problem.metadata_buffers[4] = head.generations.buffer;  // the rest is watched through the gather
  problem.error_stride = head.dispatches;
  problem.attention_error_offset = head.attention_at;
  problem.one_row_per_lane = 1;   // by construction: every member is one query row of its own lane
  if (!run_ragged_attention(b, problem, errors)) return FH_ALLOCATION_FAILED;

  for (uint32_t base = 0; base < lanes; base += kLaneChunk) {
    uint32_t chunk = std::min<uint32_t>(kLaneChunk, lanes - base);
    LaneRows targets{};
    for (uint32_t local = 0; local < chunk; ++local) {
      const LaneMember &m = run.members[base + local];
      View row;
      if ((status = make_view(b, m.out, true, &row)) != FH_OK) return status;
      targets.first[local] = row.base + row.offset * dtype_size(row.dtype);
      if (m.has_copy) {
        if ((status = make_view(b, m.copy_target, true, &row)) != FH_OK) return status;
        targets.second[local] = row.base + row.offset * dtype_size(row.dtype);
      }
    }
    launch_scatter_lane_rows(b->stream, targets, rows, base, chunk, (uint32_t)row_bytes);
  }
  b->fused_runs += 1;
  b->fused_dispatches += run.dispatches;
  return FH_OK;
}

// ---- runs that bring prefill chunks ----
// A sequence's chunk of n > 1 rows recorded on its own (the multi-row branch of
// paged_cache_attention, engines/qwen3-coder/src/lib.rs:685-707: cache.append, then
// cache.attention): two Op::PagedCopy{IntoPages} of the chunk's key and value rows and one causal
// Op::PagedSdpa over its n query rows, optionally followed by the Op::Copy that moves the
// attended rows, token-major, into the packed activation.  Such members, and one-row members in
// either idiom, next to each other are one ragged launch over the packed rows.

// rows [n, ...] whose inner axes are packed, as [n, heads, width] with its own row stride.
bool as_chunk_rows(const fh_tensor &rows, uint32_t n, uint32_t heads, uint32_t width, fh_tensor *out) {
  if (rows.rank < 2 || rows.shape[0] != n) return false;
  uint64_t inner = 1;
  for (uint32_t axis = rows.rank; axis-- > 1;) {
    if (rows.stride[axis] != inner) return false;
    inner *= rows.shape[axis];
  }
  if (inner != (uint64_t)heads * width) return false;
  *out = rows;
  out->rank = 3;
  out->shape[0] = n;
  out->shape[1] = heads;
  out->shape[2] = width;
  out->stride[1] = width;
  out->stride[2] = 1;
  return true;
}

// `copy` moves the attended rows of `out` [heads, n, width], token by token, into a destination
// [n, heads, width] whose head rows are dense.
bool copies_attended_chunk(const fh_tensor &out, const fh_dispatch &copy) {
  if (copy.op != FH_OP_COPY || copy.n_inputs != 1 || copy.n_outputs != 1) return false;
  const fh_tensor &in = copy.inputs[0], &to = copy.outputs[0];
  if (in.buffer != out.buffer || in.offset != out.offset || in.dtype != out.dtype || to.dtype != out.dtype)
    return false;
  if (in.rank != 3 || to.rank != 3) return false;
  const uint32_t shape[3] = {out.shape[1], out.shape[0], out.shape[2]};
  for (uint32_t axis = 0; axis < 3; ++axis)
    if (in.shape[axis] != shape[axis] || to.shape[axis] != shape[axis]) return false;
  if (in.stride[0] != out.stride[1] || in.stride[1] != out.stride[0] || in.stride[2] != 1) return false;
  return to.stride[2] == 1 && to.stride[1] == to.shape[2];
}

bool chunk_member_at(const fh_dispatch *d, uint32_t count, uint32_t at, LaneMember *m) {
  *m = LaneMember{};
  if (at + 2 >= count) return false;
  const fh_dispatch &first = d[at], &second = d[at + 1], &attention = d[at + 2];
  if (first.op != FH_OP_PAGED_COPY || second.op != FH_OP_PAGED_COPY || attention.op != FH_OP_PAGED_SDPA)
    return false;
  if (first.direction != 0 || second.direction != 0 || attention.causal == 0) return false;
  if (first.n_inputs != second.n_inputs || attention.n_inputs != first.n_inputs + 2) return false;
  if (attention.n_outputs != 1) return false;
  const fh_tensor &q = attention.inputs[0], &kp = attention.inputs[1], &vp = attention.inputs[2];
  const uint32_t n = q.shape[1];
  if (n < 2 || q.stride[2] != 1) return false;
  if (first.outputs[0].buffer != kp.buffer || first.outputs[0].offset != kp.offset ||
      first.outputs[0].dtype != kp.dtype || second.outputs[0].buffer != vp.buffer ||
      second.outputs[0].offset != vp.offset || second.outputs[0].dtype != vp.dtype)
    return false;
  if (first.start != attention.q_start || second.start != attention.q_start ||
      (uint64_t)attention.key_length != (uint64_t)attention.q_start + n ||
      first.page_tokens != attention.page_tokens || second.page_tokens != attention.page_tokens)
    return false;
  for (const fh_dispatch *copy : {&first, &second}) {
    if (!same_tensor(copy->inputs[1], attention.inputs[3]) || !same_tensor(copy->inputs[2], attention.inputs[4]))
      return false;
    if (copy->n_inputs == 4 && !same_tensor(copy->inputs[3], attention.inputs[5])) return false;
  }
  if (!as_chunk_rows(first.inputs[0], n, kp.shape[2], kp.shape[3], &m->k_new) ||
      !as_chunk_rows(second.inputs[0], n, vp.shape[2], vp.shape[3], &m->v_new))
    return false;
  m->q = q;
  m->table = attention.inputs[3];
  m->generations = attention.inputs[4];
  m->has_activity = attention.n_inputs == 6;
  if (m->has_activity) m->activity = attention.inputs[5];
  m->out = attention.outputs[0];
  m->key_pool = kp;
  m->value_pool = vp;
  m->q_start = attention.q_start;
  m->page_tokens = attention.page_tokens;
  m->tokens = n;
  m->scale = attention.scale;
  m->dispatches = 3;
  m->attention_at = 2;
  if (m->k_new.dtype != q.dtype || m->v_new.dtype != q.dtype) return false;
  if (m->out.stride[2] != 1 || !is_contiguous(m->table)) return false;
  if (m->has_activity && element_count(m->activity) != 1) return false;
  if (at + 3 < count && copies_attended_chunk(m->out, d[at + 3])) {
    m->has_copy = true;
    m->copy_target = d[at + 3].outputs[0];
    m->dispatches = 4;
  }
  return true;
}

// Whether `b` can follow `a` in a run with chunks: everything but the per-member row count, the
// outputs' layouts and the presence of a copy agrees.
bool same_chunk_shape(const LaneMember &a, const LaneMember &b) {
  if (a.has_activity != b.has_activity) return false;
  if (memcmp(&a.scale, &b.scale, sizeof(float)) != 0 || a.page_tokens != b.page_tokens) return false;
  const fh_tensor *left[3] = {&a.q, &a.k_new, &a.v_new}, *right[3] = {&b.q, &b.k_new, &b.v_new};
  for (uint32_t i = 0; i < 3; ++i)
    if (left[i]->buffer != right[i]->buffer || left[i]->dtype != right[i]->dtype) return false;
  // heads, widths and the distance between a row's heads
  if (a.q.shape[0] != b.q.shape[0] || a.q.shape[2] != b.q.shape[2] || a.q.stride[0] != b.q.stride[0] ||
      a.q.stride[2] != b.q.stride[2])
    return false;
  for (uint32_t i = 1; i < 3; ++i)
    if (left[i]->shape[1] != right[i]->shape[1] || left[i]->shape[2] != right[i]->shape[2] ||
        left[i]->stride[1] != right[i]->stride[1] || left[i]->stride[2] != right[i]->stride[2])
      return false;
  if (!same_layout(a.table, b.table) || !same_tensor(a.generations, b.generations)) return false;
  if (a.has_activity && !same_layout(a.activity, b.activity)) return false;
  if (a.out.dtype != b.out.dtype || a.out.shape[0] != b.out.shape[0] || a.out.shape[2] != b.out.shape[2]) return false;
  return same_tensor(a.key_pool, b.key_pool) && same_tensor(a.value_pool, b.value_pool);
}

// The elements [lo, hi) of its buffer a strided tensor touches at most.
void extent_of(const fh_tensor &t, uint64_t *lo, uint64_t *hi) {
  uint64_t last = 0;
  for (uint32_t axis = 0; axis < t.rank; ++axis)
    if (t.shape[axis] > 0) last += (uint64_t)(t.shape[axis] - 1) * t.stride[axis];
  *lo = t.offset;
  *hi = t.offset + last + 1;
}

// Most rows of attended output a run with chunks may stage, and most work of its overlap check.
constexpr uint64_t kChunkRowsBytes = 256ull << 20;
constexpr uint64_t kChunkCheckWork = 1ull << 27;

// Longest run starting at `first` that has at least two members, at least one of them a chunk, and
// whose packed rows follow each other at one row stride per tensor.  `run->delta` holds the row
// strides of q and the new key and value rows.
bool find_chunk_run(const fh_dispatch *d, uint32_t count, uint32_t first, LaneRun *run) {
  *run = LaneRun{};
  {   // nothing to look for unless the stretch of per-lane dispatches ahead holds a multi-row attention
    bool chunk_ahead = false;
    for (uint32_t at = first; at < count && !chunk_ahead; ++at) {
      const uint32_t op = d[at].op;
      if (op == FH_OP_PAGED_SDPA)
        chunk_ahead = d[at].n_inputs >= 1 && d[at].inputs[0].rank == 3 && d[at].inputs[0].shape[1] > 1;
      else if (op != FH_OP_PAGED_COPY && op != FH_OP_PAGED_SDPA_APPEND && op != FH_OP_COPY)
        break;
    }
    if (!chunk_ahead) return false;
  }
  auto member_at = [&](uint32_t at, LaneMember *m) {
    return chunk_member_at(d, count, at, m) || lane_member_at(d, count, at, m);
  };
  // row strides: known from a chunk member's own tensors, else from the first two members
  auto strides_of = [](const LaneMember &m, int64_t out[3]) {
    out[0] = (int64_t)m.q.stride[1];
    out[1] = (int64_t)m.k_new.stride[0];
    out[2] = (int64_t)m.v_new.stride[0];
  };
  LaneMember member;
  if (!member_at(first, &member)) return false;
  bool known = member.tokens > 1, any_chunk = member.tokens > 1;
  if (known) strides_of(member, run->delta);
  run->members.push_back(member);
  run->dispatches = member.dispatches;
  uint64_t tokens = member.tokens;
  for (;;) {
    const uint32_t at = first + run->dispatches;
    if (at >= count || !member_at(at, &member)) break;
    const LaneMember &head = run->members[0];
    if (!same_chunk_shape(head, member)) break;
    const fh_tensor *mine[3] = {&member.q, &member.k_new, &member.v_new};
    const fh_tensor *heads[3] = {&head.q, &head.k_new, &head.v_new};
    int64_t delta[3] = {run->delta[0], run->delta[1], run->delta[2]};
    bool regular = true;
    for (uint32_t i = 0; i < 3 && regular; ++i) {
      const int64_t distance = (int64_t)mine[i]->offset - (int64_t)heads[i]->offset;
      if (distance <= 0) regular = false;
      else if (!known) {
        if (distance % (int64_t)tokens != 0) regular = false;
        delta[i] = distance / (int64_t)tokens;
      } else if (distance != delta[i] * (int64_t)tokens) {
        regular = false;
      }
    }
    if (regular && member.tokens > 1) {
      int64_t own[3];
      strides_of(member, own);
      for (uint32_t i = 0; i < 3; ++i)
        if (own[i] != delta[i]) regular = false;
    }
    if (!regular) break;
    for (uint32_t i = 0; i < 3; ++i) run->delta[i] = delta[i];
    known = true;
    any_chunk = any_chunk || member.tokens > 1;
    tokens += member.tokens;
    run->members.push_back(member);
    run->dispatches += member.dispatches;
  }
  if (run->members.size() < 2 || !any_chunk) return false;
  const LaneMember &head = run->members[0];
  for (uint32_t i = 0; i < 3; ++i)
    if (run->delta[i] <= 0) return false;
  if (tokens * head.q.shape[0] * head.out.shape[2] * dtype_size(head.out.dtype) > kChunkRowsBytes) return false;
  // the scatter of the attended rows addresses each destination with 32-bit byte strides
  for (const LaneMember &m : run->members) {
    const uint64_t element = dtype_size(m.out.dtype);
    if (m.out.stride[0] * element >= (1ull << 32)) return false;
    if (m.tokens > 1 && m.out.stride[1] * element >= (1ull << 32)) return false;
    if (m.has_copy && m.tokens > 1 && m.copy_target.stride[0] * element >= (1ull << 32)) return false;
  }
  // the overlap check walks every reader's pages against every writer's: bounded here
  {
    uint64_t read_pages = 0, written_pages = 0;
    for (const LaneMember &m : run->members) {
      read_pages += ((uint64_t)m.q_start + m.tokens) / m.page_tokens + 1;
      written_pages += (uint64_t)m.tokens / m.page_tokens + 2;
    }
    if (read_pages * written_pages > kChunkCheckWork) return false;
  }
  // Nothing a member writes may be something another member reads or writes.
  std::unordered_set<uint64_t> read;
  for (const fh_tensor *t : {&head.q, &head.k_new, &head.v_new, &head.generations, &head.key_pool,
                             &head.value_pool})
    read.insert(t->buffer);
  struct Span {
    uint64_t buffer, lo, hi;
  };
  std::vector<Span> written;
  written.reserve(run->members.size() * 2);
  std::vector<std::pair<uint64_t, uint64_t>> tables;
  tables.reserve(run->members.size());
  for (const LaneMember &m : run->members) {
    read.insert(m.table.buffer);
    if (m.has_activity) read.insert(m.activity.buffer);
    uint64_t lo, hi;
    extent_of(m.out, &lo, &hi);
    written.push_back({m.out.buffer, lo, hi});
    if (m.has_copy) {
      extent_of(m.copy_target, &lo, &hi);
      written.push_back({m.copy_target.buffer, lo, hi});
    }
    tables.push_back({m.table.buffer, m.table.offset});
  }
  for (const Span &span : written)
    if (read.count(span.buffer)) return false;
  // Two members on one table would store into the same slots: order matters, so no fusion.
  std::sort(tables.begin(), tables.end());
  if (std::adjacent_find(tables.begin(), tables.end()) != tables.end()) return false;
  std::sort(written.begin(), written.end(), [](const Span &a, const Span &b) {
    return a.buffer != b.buffer ? a.buffer < b.buffer : a.lo < b.lo;
  });
  for (size_t i = 1; i < written.size(); ++i)
    if (written[i].buffer == written[i - 1].buffer && written[i].lo < written[i - 1].hi) return false;
  return true;
}

// Executes the run found by find_chunk_run; same contract as run_lane_group.  A member's failures
// go to the records of its own dispatches: storing a row to the first copy's (or the append's),
// attending to the attention's.
fh_status run_chunk_group(fh_backend *b, const LaneRun &run, ErrorSlot *errors, bool *executed) {
  *executed = true;
  const LaneMember &head = run.members[0];
  const fh_tensor &q0 = head.q, &kp = head.key_pool, &vp = head.value_pool;
  const uint32_t lanes = (uint32_t)run.members.size(), heads = q0.shape[0];
  const uint32_t table_pages = head.table.shape[0], table_words = table_pages * 2;
  const uint32_t out_dtype = head.out.dtype, value_width = head.out.shape[2];
  const uint64_t head_bytes = (uint64_t)value_width * dtype_size(out_dtype);
  uint64_t tokens64 = 0;
  for (const LaneMember &m : run.members) tokens64 += m.tokens;
  FH_REQUIRE(tokens64 < (1ull << 31) && head_bytes * heads < (1ull << 31));
  const uint32_t tokens = (uint32_t)tokens64;
  // tables, activity, starts, cu (+ the overlap flag), the members' record indices; staged
  // failure records of every row; the attended rows
  const uint64_t metadata_words = (uint64_t)lanes * table_words + 5ull * lanes + 2;
  const uint64_t staged_at = (metadata_words * 4 + 255) / 256 * 256;
  const uint64_t rows_at = (staged_at + 2ull * tokens * sizeof(ErrorSlot) + 255) / 256 * 256;
  char *scratch = b->ensure_lane_scratch(rows_at + (uint64_t)tokens * heads * head_bytes);
  if (!scratch) {   // no room to stage the run (a caller that may not allocate): one by one
    *executed = false;
    return FH_OK;
  }
  uint32_t *tables = (uint32_t *)scratch;
  uint32_t *activity = tables + (uint64_t)lanes * table_words;
  uint32_t *starts = activity + lanes;
  uint32_t *cu = starts + lanes;
  uint32_t *records = cu + lanes + 2;
  ErrorSlot *staged = (ErrorSlot *)(scratch + staged_at);
  char *rows = scratch + rows_at;

  std::vector<uint64_t> key;
  key.reserve(6ull * lanes + 3);
  key.push_back(~0ull);   // (a run of one-row members never has this first word: its lane count)
  key.push_back(lanes);
  key.push_back(table_words);
  for (const LaneMember &m : run.members) {
    key.push_back(m.table.buffer);
    key.push_back(m.table.offset);
    key.push_back(m.has_activity ? m.activity.buffer : 0);
    key.push_back(m.has_activity ? m.activity.offset : 0);
    key.push_back(m.q_start);
    key.push_back(((uint64_t)m.tokens << 32) | ((uint64_t)m.dispatches << 8) | m.attention_at);
  }
  fh_status status;
  if (!(b->lane_metadata_valid && key == b->lane_metadata_key)) {
    b->lane_metadata_valid = false;
    b->attention_plan_valid = false;  // the plan was built from the metadata replaced here
    b->lane_metadata_watch.clear();
    uint32_t first_token = 0, record = 0;
    for (uint32_t base = 0; base < lanes; base += kChunkMembers) {
      const uint32_t chunk = std::min<uint32_t>(kChunkMembers, lanes - base);
      ChunkSources sources{};
      for (uint32_t local = 0; local < chunk; ++local) {
        const LaneMember &m = run.members[base + local];
        View table, flag;
        if ((status = make_view(b, m.table, false, &table)) != FH_OK) return status;
        sources.table[local] = (const uint32_t *)table.base + table.offset;
        b->lane_metadata_watch.insert(m.table.buffer);
        if (m.has_activity) {
          if ((status = make_view(b, m.activity, false, &flag)) != FH_OK) return status;
          sources.activity[local] = (const uint32_t *)flag.base + flag.offset;
          b->lane_metadata_watch.insert(m.activity.buffer);
        }
        sources.start[local] = m.q_start;
        sources.first_token[local] = first_token;
        sources.append_record[local] = record;
        sources.attention_record[local] = record + m.attention_at;
        first_token += m.tokens;
        record += m.dispatches;
      }
      launch_gather_chunk_metadata(b->stream, sources, base, chunk, lanes, tokens, table_words, tables,
                                   activity, starts, cu, records);
    }
    launch_init_errors(b->stream, staged, 2 * tokens);
    // The one thing the tensors cannot show: a row stored into a slot another member attends.
    uint32_t *flag = cu + lanes + 1;
    launch_chunk_conflict_check(b->stream, tables, activity, starts, cu, lanes, table_pages,
                                head.page_tokens, flag);
    if (hipMemcpyAsync(b->host_flag, flag, sizeof(uint32_t), hipMemcpyDeviceToHost, b->stream) != hipSuccess ||
        hipStreamSynchronize(b->stream) != hipSuccess)
      return FH_DEVICE_EXECUTION_FAILED;
    b->lane_conflict = *b->host_flag != 0;
    b->lane_metadata_key = std::move(key);
    b->lane_metadata_valid = true;
  }
  if (b->lane_conflict) {
    *executed = false;
    return FH_OK;
  }

  auto device_view = [](char *base, uint32_t dtype, std::initializer_list<uint32_t> shape) {
    View v{};
    v.base = base;
    v.dtype = dtype;
    v.rank = (uint32_t)shape.size();
    for (uint32_t axis = 0; axis < FH_MAX_RANK; ++axis) {
      v.shape[axis] = 1;
      v.stride[axis] = 0;
    }
    uint32_t axis = 0;
    for (uint32_t extent : shape) v.shape[axis++] = extent;
    uint64_t stride = 1;
    for (int at = (int)v.rank - 1; at >= 0; --at) {
      v.stride[at] = stride;
      stride *= v.shape[at];
    }
    return v;
  };
  RaggedAttention problem{};
  // q [heads, n, D] per member -> [tokens, heads, D]; new rows [n, Hkv, D] -> [tokens, Hkv, D]
  if ((status = make_view(b, q0, false, &problem.q)) != FH_OK) return status;
  problem.q.shape[0] = tokens;
  problem.q.shape[1] = heads;
  problem.q.stride[0] = (uint64_t)run.delta[0];
  problem.q.stride[1] = q0.stride[0];
  View *appended[2] = {&problem.k_new, &problem.v_new};
  const fh_tensor *appended_from[2] = {&head.k_new, &head.v_new};
  for (uint32_t i = 0; i < 2; ++i) {
    if ((status = make_view(b, *appended_from[i], false, appended[i])) != FH_OK) return status;
    appended[i]->shape[0] = tokens;
    appended[i]->stride[0] = (uint64_t)run.delta[1 + i];
  }
  if ((status = make_view(b, head.generations, false, &problem.generations)) != FH_OK) return status;
  if ((status = make_view(b, kp, true, &problem.key_pool)) != FH_OK) return status;
  if ((status = make_view(b, vp, true, &problem.value_pool)) != FH_OK) return status;
  problem.tables = device_view((char *)tables, FH_U32, {lanes, table_pages, 2});
  problem.activity = device_view((char *)activity, FH_U32, {lanes});
  problem.q_starts = device_view((char *)starts, FH_U32, {lanes});
  problem.cu_seqlens = device_view((char *)cu, FH_U32, {lanes + 1});
  problem.out = device_view(rows, out_dtype, {tokens, heads, value_width});
  problem.tokens = tokens;
  problem.lanes = lanes;
  problem.query_heads = heads;
  problem.kv_heads = kp.shape[2];
  problem.width = q0.shape[2];
  problem.value_width = value_width;
  problem.page_tokens = head.page_tokens;
  problem.physical_pages = kp.shape[0];
  problem.table_pages = table_pages;
  problem.scale = head.scale;
  problem.metadata_buffers[4] = head.generations.buffer;  // the rest is watched through the gather
  problem.error_stride = 2;             // staged records: (storing, attending) per row
  problem.attention_error_offset = 1;
  problem.one_row_per_lane = 0;
  if (!run_ragged_attention(b, problem, staged)) {
    b->lane_metadata_valid = false;
    return FH_ALLOCATION_FAILED;
  }
  launch_fold_chunk_errors(b->stream, staged, errors, cu, records, lanes, tokens);

  const uint32_t element = dtype_size(out_dtype);
  uint32_t first_token = 0;
  for (uint32_t base = 0; base < lanes; base += kChunkMembers) {
    const uint32_t chunk = std::min<uint32_t>(kChunkMembers, lanes - base);
    ChunkTargets targets{};
    for (uint32_t local = 0; local < chunk; ++local) {
      const LaneMember &m = run.members[base + local];
      View rows_view;
      if ((status = make_view(b, m.out, true, &rows_view)) != FH_OK) return status;
      targets.target[0][local] = rows_view.base + rows_view.offset * element;
      targets.token_stride[0][local] = m.tokens > 1 ? (uint32_t)(m.out.stride[1] * element) : 0;   // out is [heads, n, width]
      targets.head_stride[0][local] = (uint32_t)(m.out.stride[0] * element);
      if (m.has_copy) {
        if ((status = make_view(b, m.copy_target, true, &rows_view)) != FH_OK) return status;
        targets.target[1][local] = rows_view.base + rows_view.offset * element;
        if (m.tokens > 1) {   // [n, heads, width], head rows dense
          targets.token_stride[1][local] = (uint32_t)(m.copy_target.stride[0] * element);
        } else {              // one dense row of heads * width elements
          targets.token_stride[1][local] = 0;
        }
        targets.head_stride[1][local] = (uint32_t)head_bytes;
      }
      targets.first_token[local] = first_token;
      first_token += m.tokens;
    }
    targets.first_token[chunk] = first_token;
    launch_scatter_chunk_rows(b->stream, targets, rows, chunk, heads, (uint32_t)head_bytes);
  }
  b->fused_runs += 1;
  b->fused_dispatches += run.dispatches;
  return FH_OK;
}

// The BackendError a raised error record of dispatch `index` (operation `op`) stands for.
fh_status failure_of(uint32_t op, uint32_t index, uint64_t serial, const ErrorSlot &record,
                     fh_error *error) {
  const bool index_error = op == FH_OP_GATHER_QUANT_MATMUL || op == FH_OP_QUANT_EMBED ||
                           op == FH_OP_ROUTE_PACK;
  // Sampling refuses its live parameters or mask as InvalidInput (lib.rs:1560-1567, 1639-1652).
  const bool refused_input = op == FH_OP_SAMPLE || op == FH_OP_SAMPLE_MASKED;
  const fh_status result = refused_input ? FH_INVALID_INPUT
                                         : (index_error ? FH_INDEX_OUT_OF_RANGE : FH_DEVICE_ERROR_FLAG);
  error->code = result;
  error->dispatch = index;
  error->submission = serial;
  error->operation = op;
  error->flag = record.flag;
  error->value = record.value;
  return result;
}

hipEvent_t take_event(fh_backend *b) {
  if (!b->event_pool.empty()) {
    hipEvent_t e = b->event_pool.back();
    b->event_pool.pop_back();
    return e;
  }
  hipEvent_t e = nullptr;
  (void)hipEventCreate(&e);
  return e;
}

// Returns a finished submission's error record and events to the backend's pools.
void recycle_submission(fh_backend *b, fh_submission *s) {
  if (s->device_errors)
    b->error_pool.push_back({s->device_errors, s->host_errors, s->error_capacity});
  if (s->start) b->event_pool.push_back(s->start);
  if (s->end) b->event_pool.push_back(s->end);
  if (s->done) b->event_pool.push_back(s->done);
  for (auto &span : s->spans) {
    b->event_pool.push_back(span.begin);
    b->event_pool.push_back(span.finish);
  }
  s->spans.clear();
  s->device_errors = nullptr;
  s->host_errors = nullptr;
  s->start = s->end = s->done = nullptr;
}

void drain_profile(fh_backend *b) {
  for (auto &t : b->timed) {
    float ms = 0.0f;
    if (hipEventElapsedTime(&ms, t.start, t.end) == hipSuccess) {
      b->class_ns[t.kernel_class] += (uint64_t)((double)ms * 1e6);
      b->class_launches[t.kernel_class] += 1;
    }
    b->event_pool.push_back(t.start);
    b->event_pool.push_back(t.end);
  }
  b->timed.clear();
}

}  // namespace

// ================================================================== C ABI

extern "C" {

const char *fh_version(void) { return "forja-hip 0.1 (gfx950)"; }

fh_status fh_create(int device, fh_backend **out) {
  if (!out) return FH_INVALID_INPUT;
  *out = nullptr;
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || device < 0 || device >= count)
    return FH_DEVICE_EXECUTION_FAILED;
  fh_backend *b = new (std::nothrow) fh_backend();
  if (!b) return FH_ALLOCATION_FAILED;
  b->device = device;
  if (hipSetDevice(device) != hipSuccess || hipGetDeviceProperties(&b->props, device) != hipSuccess ||
      hipStreamCreate(&b->stream) != hipSuccess) {
    delete b;
    return FH_DEVICE_EXECUTION_FAILED;
  }
  // fh_submit_static may allocate nothing, so what it needs is set up here: this device's address
  // of the fixed scratch array and a pinned mirror of its error records.
  b->static_scratch = static_scratch_address(device);
  void *mirror = nullptr;
  if (!b->static_scratch ||
      hipHostMalloc(&mirror, kStaticErrorBytes, hipHostMallocDefault) != hipSuccess) {
    (void)hipStreamDestroy(b->stream);
    delete b;
    return FH_DEVICE_EXECUTION_FAILED;
  }
  b->static_host_errors = (ErrorSlot *)mirror;
  void *word = nullptr;
  if (hipHostMalloc(&word, 64, hipHostMallocDefault) != hipSuccess) {
    (void)hipHostFree(mirror);
    (void)hipStreamDestroy(b->stream);
    delete b;
    return FH_DEVICE_EXECUTION_FAILED;
  }
  b->host_flag = (uint32_t *)word;
  {
    std::lock_guard<std::mutex> lock(g_live_mutex);
    g_live_backends.insert(b);
  }
  *out = b;
  return FH_OK;
}

void fh_destroy(fh_backend *b) {
  if (!b) return;
  {
    std::lock_guard<std::mutex> lock(g_live_mutex);
    if (!g_live_backends.erase(b)) return;
  }
  {
    std::lock_guard<std::mutex> lock(b->mutex);
    (void)hipSetDevice(b->device);
    (void)hipStreamSynchronize(b->stream);
    for (fh_submission *s : b->submissions) {
      (void)hipFree(s->device_errors);
      (void)hipHostFree(s->host_errors);
      (void)hipEventDestroy(s->start);
      (void)hipEventDestroy(s->end);
      (void)hipEventDestroy(s->done);
      s->device_errors = nullptr;
      s->host_errors = nullptr;
    }
    b->submissions.clear();
    for (auto &entry : b->allocations) (void)hipFree(entry.second.ptr);
    for (auto &entry : b->programs)
      for (auto &typed : entry.second.typed) (void)hipFree(typed.second);
    if (b->workspace) (void)hipFree(b->workspace);
    if (b->accumulators) (void)hipFree(b->accumulators);
    if (b->lane_scratch) (void)hipFree(b->lane_scratch);
    if (b->route_plan) (void)hipFree(b->route_plan);
    if (b->attention_plan) (void)hipFree(b->attention_plan);
    for (auto &e : b->prepared) (void)hipFree(e.operand);
    for (auto &e : b->dead_prepared) (void)hipFree(e.operand);
    for (auto &e : b->error_pool) {
      (void)hipFree(e.device);
      (void)hipHostFree(e.host);
    }
    if (b->ring) (void)hipHostFree(b->ring);
    if (b->static_host_errors) (void)hipHostFree(b->static_host_errors);
    if (b->host_flag) (void)hipHostFree(b->host_flag);
    for (auto &open : b->open_timers)
      for (auto e : open) (void)hipEventDestroy(e);
    for (auto &t : b->timed) {
      (void)hipEventDestroy(t.start);
      (void)hipEventDestroy(t.end);
    }
    for (auto e : b->event_pool) (void)hipEventDestroy(e);
    (void)hipStreamDestroy(b->stream);
  }
  delete b;
}

static fh_status alloc_locked(fh_backend *b, uint64_t bytes, bool readonly, fh_buffer *out) {
  void *ptr = nullptr;
  uint64_t want = bytes == 0 ? 256 : bytes;
  b->reap_dead_prepared();
  // the quota covers the caller's allocations and what the library keeps for them; what it keeps
  // goes before an allocation is refused
  if (b->memory_limit && b->used_bytes + b->prepared_bytes + bytes > b->memory_limit) b->evict_prepared();
  if (b->memory_limit && b->used_bytes + b->prepared_bytes + bytes > b->memory_limit) return FH_QUOTA_EXCEEDED;
  if (hipMalloc(&ptr, want) != hipSuccess) {
    (void)hipGetLastError();
    if (!b->evict_prepared() || hipMalloc(&ptr, want) != hipSuccess) {
      (void)hipGetLastError();
      return FH_ALLOCATION_FAILED;
    }
  }
  if (hipMemsetAsync(ptr, 0, want, b->stream) != hipSuccess) {
    (void)hipFree(ptr);
    return FH_DEVICE_EXECUTION_FAILED;
  }
  uint64_t id = b->next_id++;
  b->allocations[id] = Allocation{(char *)ptr, bytes, readonly};
  b->used_bytes += bytes;
  *out = id;
  return FH_OK;
}

fh_status fh_alloc(fh_backend *b, uint64_t bytes, fh_buffer *out) {
  if (!b || !out) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  (void)hipSetDevice(b->device);
  return alloc_locked(b, bytes, false, out);
}

fh_status fh_release(fh_backend *b, fh_buffer buffer) {
  if (!b) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  auto it = b->allocations.find(buffer);
  if (it == b->allocations.end()) return FH_INVALID_INPUT;
  (void)hipSetDevice(b->device);
  (void)hipStreamSynchronize(b->stream);
  b->reap_dead_prepared();
  b->drop_prepared(buffer);
  (void)hipFree(it->second.ptr);
  b->used_bytes -= it->second.bytes;
  b->allocations.erase(it);
  return FH_OK;
}

fh_status fh_import(fh_backend *b, const void *bytes, uint64_t len, fh_buffer *out) {
  if (!b || !out || (!bytes && len)) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  (void)hipSetDevice(b->device);
  fh_status status = alloc_locked(b, len, true, out);
  if (status != FH_OK) return status;
  if (len && hipMemcpyAsync(b->allocations[*out].ptr, bytes, len, hipMemcpyHostToDevice,
                            b->stream) != hipSuccess)
    return FH_DEVICE_EXECUTION_FAILED;
  if (hipStreamSynchronize(b->stream) != hipSuccess) return FH_DEVICE_EXECUTION_FAILED;
  return FH_OK;
}

fh_status fh_write(fh_backend *b, fh_buffer buffer, uint64_t byte_offset, const void *bytes,
                   uint64_t len) {
  if (!b || (!bytes && len)) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  auto it = b->allocations.find(buffer);
  if (it == b->allocations.end() || it->second.readonly) return FH_INVALID_INPUT;
  if (byte_offset > it->second.bytes || len > it->second.bytes - byte_offset)
    return FH_INVALID_INPUT;
  if (len == 0) return FH_OK;
  (void)hipSetDevice(b->device);
  b->reap_dead_prepared();
  b->drop_prepared(buffer);
  // Small writes are staged through a pinned ring and ordered on the stream without waiting for
  // it; the caller's bytes may be reused as soon as this returns either way.
  constexpr uint64_t kRingBytes = 32ull << 20, kRingPiece = 4ull << 20;
  if (len <= kRingPiece) {
    if (!b->ring) {
      void *ptr = nullptr;
      if (hipHostMalloc(&ptr, kRingBytes, hipHostMallocDefault) == hipSuccess) {
        b->ring = (char *)ptr;
        b->ring_bytes = kRingBytes;
        b->ring_head = 0;
      }
    }
    if (b->ring) {
      uint64_t need = (len + 255) / 256 * 256;
      if (b->ring_head + need > b->ring_bytes) {
        // Wrap: every earlier staged copy must have left the ring.
        if (hipStreamSynchronize(b->stream) != hipSuccess) return FH_DEVICE_EXECUTION_FAILED;
        b->ring_head = 0;
      }
      char *stage = b->ring + b->ring_head;
      memcpy(stage, bytes, len);
      b->ring_head += need;
      if (hipMemcpyAsync(it->second.ptr + byte_offset, stage, len, hipMemcpyHostToDevice,
                         b->stream) != hipSuccess)
        return FH_DEVICE_EXECUTION_FAILED;
      return FH_OK;
    }
  }
  if (hipMemcpyAsync(it->second.ptr + byte_offset, bytes, len, hipMemcpyHostToDevice, b->stream) !=
      hipSuccess)
    return FH_DEVICE_EXECUTION_FAILED;
  if (hipStreamSynchronize(b->stream) != hipSuccess) return FH_DEVICE_EXECUTION_FAILED;
  return FH_OK;
}

fh_status fh_read(fh_backend *b, fh_buffer buffer, uint64_t byte_offset, void *bytes,
                  uint64_t len) {
  if (!b || (!bytes && len)) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  auto it = b->allocations.find(buffer);
  if (it == b->allocations.end()) return FH_INVALID_INPUT;
  if (byte_offset > it->second.bytes || len > it->second.bytes - byte_offset)
    return FH_INVALID_INPUT;
  if (len == 0) return FH_OK;
  (void)hipSetDevice(b->device);
  if (hipMemcpyAsync(bytes, it->second.ptr + byte_offset, len, hipMemcpyDeviceToHost, b->stream) !=
      hipSuccess)
    return FH_DEVICE_EXECUTION_FAILED;
  if (hipStreamSynchronize(b->stream) != hipSuccess) return FH_DEVICE_EXECUTION_FAILED;
  return FH_OK;
}

fh_status fh_read_tensor(fh_backend *b, const fh_tensor *tensor, void *bytes, uint64_t len) {
  if (!b || !tensor || (!bytes && len)) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  (void)hipSetDevice(b->device);
  View view;
  fh_status status = make_view(b, *tensor, false, &view);
  if (status != FH_OK) return status;
  uint64_t elements = element_count(*tensor);
  uint64_t size = dtype_size(tensor->dtype);
  if (len != elements * size) return FH_INVALID_INPUT;
  if (elements == 0) return FH_OK;
  char *staging = b->ensure_workspace(elements * size);
  if (!staging) return FH_ALLOCATION_FAILED;
  // Gather on the device as a same-dtype copy into contiguous staging.
  View flat = contiguous_view(staging, tensor->dtype, *tensor);
  View source = view;
  if (tensor->dtype == FH_I32) {
    source.dtype = FH_U32;
    flat.dtype = FH_U32;
  }
  if (is_float(tensor->dtype) && tensor->dtype != FH_F32) {
    // 16-bit payloads are moved as raw bits by viewing them as u16 pairs is not possible with
    // arbitrary strides; the float path round-trips exactly (f16/bf16 -> f32 -> same dtype).
  }
  launch_copy(b->stream, source, flat, elements);
  if (hipMemcpyAsync(bytes, staging, elements * size, hipMemcpyDeviceToHost, b->stream) !=
      hipSuccess)
    return FH_DEVICE_EXECUTION_FAILED;
  if (hipStreamSynchronize(b->stream) != hipSuccess) return FH_DEVICE_EXECUTION_FAILED;
  return FH_OK;
}

fh_status fh_prepare_program(fh_backend *b, uint32_t kind, const fh_inst *insts, uint32_t n_insts,
                             const uint32_t *outputs, uint32_t n_pairs, fh_program *out) {
  if (!b || !insts || !outputs || !out) return FH_INVALID_INPUT;
  if (kind > 1 || n_insts == 0 || n_insts > 256 || n_pairs == 0 || n_pairs > kMaxProgramOutputs)
    return FH_INVALID_INPUT;
  Program p;
  p.kind = kind;
  p.insts.assign(insts, insts + n_insts);
  p.pairs.assign(outputs, outputs + 2 * n_pairs);
  uint32_t max_input = 0, max_output = 0;
  bool any_input = false;
  for (const fh_inst &inst : p.insts) {
    if (inst.kind > 8) return FH_INVALID_INPUT;
    if (inst.kind == 0) {
      if (inst.a >= kMaxProgramInputs) return FH_INVALID_INPUT;
      max_input = std::max(max_input, inst.a);
      any_input = true;
    }
    if (inst.kind == 8) {
      if (kind != 1) return FH_INVALID_INPUT;
      p.n_reduce += 1;
    }
  }
  if (p.n_reduce > kMaxReductions) return FH_INVALID_INPUT;
  std::vector<bool> seen(kMaxProgramOutputs, false);
  for (uint32_t pair = 0; pair < n_pairs; ++pair) {
    uint32_t slot = outputs[2 * pair];
    if (slot >= kMaxProgramOutputs || seen[slot] || outputs[2 * pair + 1] >= n_insts)
      return FH_INVALID_INPUT;
    seen[slot] = true;
    max_output = std::max(max_output, slot);
  }
  p.n_inputs = any_input ? max_input + 1 : 0;
  p.n_outputs = max_output + 1;
  for (uint32_t slot = 0; slot < p.n_outputs; ++slot)
    if (!seen[slot]) return FH_INVALID_INPUT;
  // validate_structure (program.rs:1052-1094): operands defined earlier, reductions only in row
  // programs and at most four.  These do not depend on how the inputs are bound.
  {
    uint32_t reductions = 0;
    for (uint32_t i = 0; i < n_insts; ++i) {
      const fh_inst &inst = p.insts[i];
      const uint32_t operands = inst.kind == 4 || inst.kind == 7 || inst.kind == 8 ? 1
                                : inst.kind == 5 ? 2 : inst.kind == 6 ? 3 : 0;
      const uint32_t values[3] = {inst.a, inst.b, inst.c};
      for (uint32_t o = 0; o < operands; ++o)
        if (values[o] >= i) return FH_INVALID_INPUT;
      if (inst.kind == 8 && (kind != 1 || ++reductions > (uint32_t)kMaxReductions))
        return FH_INVALID_INPUT;
    }
  }
  // Typing check with every input assumed f32; u32 bindings are re-typed at dispatch.
  DInst typed[kMaxProgramInsts];
  fh_status status = type_program(p, 0, FH_MAX_RANK, typed);
  if (status != FH_OK) {
    // A program whose integer inputs make the all-f32 typing fail is still legal; defer.
    bool uses_index_math = false;
    for (const fh_inst &inst : p.insts)
      if (inst.kind == 0) uses_index_math = true;
    if (!uses_index_math) return status;
  }
  p.fast = classify_program(kind, p.insts.data(), n_insts, p.pairs.data(), n_pairs);
  p.add_epilogue = kind == 0 && is_add_epilogue(p.insts, p.pairs);
  p.swiglu_epilogue = kind == 0 && is_swiglu_epilogue(p.insts, p.pairs);
  std::lock_guard<std::mutex> lock(b->mutex);
  uint64_t id = b->next_id++;
  b->programs[id] = std::move(p);
  *out = id;
  return FH_OK;
}

fh_status fh_release_program(fh_backend *b, fh_program program) {
  if (!b) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  auto it = b->programs.find(program);
  if (it == b->programs.end()) return FH_INVALID_INPUT;
  (void)hipSetDevice(b->device);
  (void)hipStreamSynchronize(b->stream);
  for (auto &typed : it->second.typed) (void)hipFree(typed.second);
  b->programs.erase(it);
  return FH_OK;
}

static fh_status submit_locked(fh_backend *b, const fh_dispatch *dispatches, uint32_t count, bool profiled,
                               fh_submission **out);

fh_status fh_submit(fh_backend *b, const fh_dispatch *dispatches, uint32_t count,
                    fh_submission **out) {
  if (!b || !out || (!dispatches && count)) return FH_INVALID_INPUT;
  *out = nullptr;
  std::lock_guard<std::mutex> lock(b->mutex);
  (void)hipSetDevice(b->device);
  return submit_locked(b, dispatches, count, false, out);
}

fh_status fh_submit_profiled(fh_backend *b, const fh_dispatch *dispatches, uint32_t count,
                             fh_submission **out) {
  if (!b || !out || (!dispatches && count)) return FH_INVALID_INPUT;
  *out = nullptr;
  std::lock_guard<std::mutex> lock(b->mutex);
  (void)hipSetDevice(b->device);
  return submit_locked(b, dispatches, count, true, out);
}

fh_status fh_submission_profile(fh_submission *s, fh_dispatch_timing *out, uint32_t capacity, uint32_t *n) {
  if (!s || !n || (!out && capacity)) return FH_INVALID_INPUT;
  if (!s->waited) return FH_INVALID_INPUT;   // the timeline exists once the submission has been waited for
  *n = (uint32_t)s->timings.size();
  for (uint32_t i = 0; i < *n && i < capacity; ++i) out[i] = s->timings[i];
  return FH_OK;
}

static fh_status submit_locked(fh_backend *b, const fh_dispatch *dispatches, uint32_t count, bool profiled,
                               fh_submission **out) {
  b->reap_dead_prepared();
  // Validate the whole list before anything is enqueued (lib.rs:1423-1432).
  for (uint32_t i = 0; i < count; ++i) {
    fh_status status = process(b, dispatches[i], nullptr, false);
    if (status != FH_OK) return status;
  }
  fh_submission *s = new (std::nothrow) fh_submission();
  if (!s) return FH_ALLOCATION_FAILED;
  s->backend = b;
  s->serial = b->next_serial++;
  s->count = count;
  s->profiled = profiled;
  s->ops.resize(count);
  uint32_t slots = count == 0 ? 1 : count;
  bool pooled = false;
  for (size_t i = 0; i < b->error_pool.size(); ++i) {
    if (b->error_pool[i].capacity >= slots) {
      s->device_errors = b->error_pool[i].device;
      s->host_errors = b->error_pool[i].host;
      s->error_capacity = b->error_pool[i].capacity;
      b->error_pool.erase(b->error_pool.begin() + (long)i);
      pooled = true;
      break;
    }
  }
  if (!pooled) {
    void *dev = nullptr, *host = nullptr;
    uint32_t capacity = std::max<uint32_t>(slots, 1024);
    if (hipMalloc(&dev, capacity * sizeof(ErrorSlot)) != hipSuccess ||
        hipHostMalloc(&host, capacity * sizeof(ErrorSlot), hipHostMallocDefault) != hipSuccess) {
      if (dev) (void)hipFree(dev);
      if (host) (void)hipHostFree(host);
      delete s;
      return FH_ALLOCATION_FAILED;
    }
    s->device_errors = (ErrorSlot *)dev;
    s->host_errors = (ErrorSlot *)host;
    s->error_capacity = capacity;
  }
  s->start = take_event(b);
  s->end = take_event(b);
  s->done = take_event(b);
  b->route_plan_valid = false;  // host writes between submissions are not tracked
  b->attention_plan_valid = false;
  launch_init_errors(b->stream, s->device_errors, slots);
  (void)hipEventRecord(s->start, b->stream);
  b->lane_metadata_valid = false;
  // Plans and gathered metadata kept between dispatches die when a dispatch writes their source.
  auto note_outputs = [b](const fh_dispatch &d) {
    for (uint32_t o = 0; o < d.n_outputs && o < FH_MAX_OUTPUTS; ++o) {
      uint64_t written = d.outputs[o].buffer;
      b->drop_prepared(written);
      if (b->route_plan_valid && written == b->route_plan_key.buffer) b->route_plan_valid = false;
      if (b->attention_plan_valid)
        for (uint64_t watched : b->attention_plan_key.buffers)
          if (watched != 0 && written == watched) b->attention_plan_valid = false;
      if (b->lane_metadata_valid && b->lane_metadata_watch.count(written))
        b->lane_metadata_valid = false;
    }
  };
  fh_status status = FH_OK;
  uint32_t no_run_before = 0;  // dispatches already examined as part of a run that was refused
  for (uint32_t i = 0; i < count && status == FH_OK;) {
    uint32_t consumed = 1;
    LaneRun run;
    const uint32_t op = dispatches[i].op;
    const bool candidate = b->lane_fusion && (op == FH_OP_PAGED_SDPA_APPEND || op == FH_OP_PAGED_COPY) &&
                           i >= no_run_before;
    // a run that brings prefill chunks first (it takes one-row members too), else one of one-row members
    const bool with_chunks = candidate && find_chunk_run(dispatches, count, i, &run);
    bool fused = with_chunks || (candidate && find_lane_run(dispatches, count, i, &run));
    if (fused)
      consumed = run.dispatches;
    else if (run.members.size() > 1)
      no_run_before = i + run.dispatches;
    for (uint32_t member = 0; member < consumed; ++member) s->ops[i + member] = dispatches[i + member].op;
    hipEvent_t t0 = nullptr, t1 = nullptr;
    if (b->profiling >= 2 || profiled) {
      t0 = take_event(b);
      t1 = take_event(b);
      (void)hipEventRecord(t0, b->stream);
    }
    if (fused) {
      bool executed = true;
      status = with_chunks ? run_chunk_group(b, run, &s->device_errors[i], &executed)
                           : run_lane_group(b, run, &s->device_errors[i], &executed);
      if (!executed) {
        fused = false;
        for (uint32_t member = 0; member < consumed && status == FH_OK; ++member) {
          status = process(b, dispatches[i + member], &s->device_errors[i + member], true);
          note_outputs(dispatches[i + member]);
        }
      }
    } else {
      NormTail tail;
      bool tail_taken = false;
      if (op == FH_OP_GATHER_QUANT_MATMUL && i + 1 < count &&
          find_norm_tail(b, dispatches[i], dispatches[i + 1], &tail)) {
        b->norm_tail = &tail;
        b->norm_tail_taken = &tail_taken;
      }
      status = process(b, dispatches[i], &s->device_errors[i], true);
      b->norm_tail = nullptr;
      b->norm_tail_taken = nullptr;
      if (tail_taken) {   // the next dispatch has been executed with this one
        consumed = 2;
        s->ops[i + 1] = dispatches[i + 1].op;
      }
    }
    for (uint32_t member = 0; member < consumed; ++member) note_outputs(dispatches[i + member]);
    if (t1) {
      (void)hipEventRecord(t1, b->stream);
      if (profiled)
        s->spans.push_back({i, consumed, dispatches[i].op, t0, t1});
      else
        b->timed.push_back({t0, t1, fused ? (uint32_t)FH_KC_ATTENTION : kernel_class_of(dispatches[i].op)});
    }
    i += consumed;
  }
  (void)hipEventRecord(s->end, b->stream);
  (void)hipMemcpyAsync(s->host_errors, s->device_errors, slots * sizeof(ErrorSlot),
                       hipMemcpyDeviceToHost, b->stream);
  (void)hipEventRecord(s->done, b->stream);
  if (status != FH_OK) {
    (void)hipStreamSynchronize(b->stream);
    recycle_submission(b, s);
    delete s;
    return status;
  }
  hipError_t launch_error = hipGetLastError();
  if (launch_error != hipSuccess) {
    s->result = FH_DEVICE_EXECUTION_FAILED;
    s->error.code = FH_DEVICE_EXECUTION_FAILED;
    s->error.submission = s->serial;
    s->error.value = (uint32_t)launch_error;
  }
  b->submissions.insert(s);
  *out = s;
  return FH_OK;
}

fh_status fh_submit_static(fh_backend *b, const fh_dispatch *dispatches, uint32_t count,
                           fh_error *error) {
  if (!b || (!dispatches && count)) return FH_INVALID_INPUT;
  if (error) memset(error, 0, sizeof(*error));
  auto fail = [&](fh_status status, uint32_t index) {
    if (error) {
      error->code = status;
      error->dispatch = index;
    }
    return status;
  };
  if ((uint64_t)count * sizeof(ErrorSlot) > kStaticErrorBytes) return fail(FH_QUOTA_EXCEEDED, count);
  std::lock_guard<std::mutex> lock(b->mutex);
  (void)hipSetDevice(b->device);
  // From here on no allocator may run: scratch needs beyond the fixed regions fail instead.
  struct Regions {
    char *workspace, *accumulators, *route_plan, *attention_plan;
    uint64_t workspace_bytes, accumulator_bytes, route_plan_bytes, attention_plan_bytes;
    int profiling;
  } saved{b->workspace, b->accumulators, b->route_plan, b->attention_plan, b->workspace_bytes,
          b->accumulator_bytes, b->route_plan_bytes, b->attention_plan_bytes, b->profiling};
  b->static_mode = true;
  b->static_overflow = false;
  b->static_programs = nullptr;
  b->static_programs_used = 0;
  b->profiling = 0;   // the timers take events from a pool that grows by allocation
  auto leave = [&] {
    b->workspace = saved.workspace;
    b->accumulators = saved.accumulators;
    b->route_plan = saved.route_plan;
    b->attention_plan = saved.attention_plan;
    b->workspace_bytes = saved.workspace_bytes;
    b->accumulator_bytes = saved.accumulator_bytes;
    b->route_plan_bytes = saved.route_plan_bytes;
    b->attention_plan_bytes = saved.attention_plan_bytes;
    b->profiling = saved.profiling;
    b->static_mode = false;
    b->static_programs = nullptr;
    b->route_plan_valid = false;   // the plans lived in the fixed array
    b->attention_plan_valid = false;
    b->lane_metadata_valid = false;
  };
  // Validate the whole list before anything is enqueued, as fh_submit does.
  for (uint32_t i = 0; i < count; ++i) {
    fh_status status = process(b, dispatches[i], nullptr, false);
    if (status != FH_OK) {
      leave();
      return fail(status, i);
    }
  }
  char *at = b->static_scratch;
  ErrorSlot *records = (ErrorSlot *)at;
  at += kStaticErrorBytes;
  b->static_programs = at;
  at += kStaticProgramBytes;
  b->route_plan = at;
  b->route_plan_bytes = kStaticRoutePlanBytes;
  at += kStaticRoutePlanBytes;
  b->attention_plan = at;
  b->attention_plan_bytes = kStaticAttentionPlanBytes;
  at += kStaticAttentionPlanBytes;
  b->accumulators = at;
  b->accumulator_bytes = kStaticAccumulatorBytes;
  at += kStaticAccumulatorBytes;
  b->workspace = at;
  b->workspace_bytes = kStaticWorkspaceBytes;
  b->route_plan_valid = false;
  b->attention_plan_valid = false;
  b->lane_metadata_valid = false;
  const uint32_t slots = count == 0 ? 1 : count;
  // The array keeps the previous call's contents: the error records must start clear (a fill
  // kernel, so that a caller may capture this call into a graph); every other region is written
  // by the kernels that read it.
  launch_init_errors(b->stream, records, slots);
  fh_status status = FH_OK;
  uint32_t index = 0;
  for (; index < count; ++index) {
    const fh_dispatch &d = dispatches[index];
    status = process(b, d, &records[index], true);
    if (status != FH_OK) break;
    for (uint32_t o = 0; o < d.n_outputs && o < FH_MAX_OUTPUTS; ++o) {
      const uint64_t written = d.outputs[o].buffer;
      b->drop_prepared(written);
      if (b->route_plan_valid && written == b->route_plan_key.buffer) b->route_plan_valid = false;
      if (b->attention_plan_valid)
        for (uint64_t watched : b->attention_plan_key.buffers)
          if (watched != 0 && written == watched) b->attention_plan_valid = false;
    }
  }
  const bool overflow = b->static_overflow;
  leave();
  if (status != FH_OK)   // a need beyond the fixed array is a quota, not an out-of-memory
    return fail(status == FH_ALLOCATION_FAILED && overflow ? FH_QUOTA_EXCEEDED : status, index);
  if (hipGetLastError() != hipSuccess) return fail(FH_DEVICE_EXECUTION_FAILED, 0);
  if (!error) return FH_OK;   // enqueued; the caller does not want to wait
  if (hipMemcpyAsync(b->static_host_errors, records, slots * sizeof(ErrorSlot),
                     hipMemcpyDeviceToHost, b->stream) != hipSuccess ||
      hipStreamSynchronize(b->stream) != hipSuccess)
    return fail(FH_DEVICE_EXECUTION_FAILED, 0);
  for (uint32_t i = 0; i < count; ++i)
    if (b->static_host_errors[i].flag)
      return failure_of(dispatches[i].op, i, 0, b->static_host_errors[i], error);
  return FH_OK;
}

fh_status fh_wait(fh_submission *s, uint64_t timeout_ns, fh_error *error) {
  if (!s) return FH_INVALID_INPUT;
  fh_backend *b = s->backend;
  if (!s->waited && !backend_alive(b)) {
    // fh_destroy drained the stream, but the error record went with the backend.
    s->waited = true;
    s->result = FH_EXECUTION_FAILED;
  }
  if (!s->waited) {
    // The event behind the trailing copy of the error records is this submission's completion
    // (Submission::wait is per submission, crates/forja-core/src/backend.rs:609-647): work
    // submitted later neither delays the wait nor counts against its deadline.
    if (timeout_ns != 0) {
      auto deadline = std::chrono::steady_clock::now() + std::chrono::nanoseconds(timeout_ns);
      for (;;) {
        hipError_t q;
        {
          std::lock_guard<std::mutex> lock(b->mutex);
          (void)hipSetDevice(b->device);
          q = hipEventQuery(s->done);
        }
        if (q == hipSuccess) break;
        if (q != hipErrorNotReady) {
          s->result = FH_DEVICE_EXECUTION_FAILED;
          break;
        }
        if (std::chrono::steady_clock::now() >= deadline) {
          if (error) {
            memset(error, 0, sizeof(*error));
            error->code = FH_TIMEOUT;
            error->submission = s->serial;
          }
          return FH_TIMEOUT;
        }
        std::this_thread::sleep_for(std::chrono::microseconds(50));
      }
    }
    // Waiting happens outside the backend's mutex, so that other threads keep submitting.
    {
      std::lock_guard<std::mutex> lock(b->mutex);
      (void)hipSetDevice(b->device);
    }
    hipError_t sync = hipEventSynchronize(s->done);
    std::lock_guard<std::mutex> lock(b->mutex);
    (void)hipSetDevice(b->device);
    s->waited = true;
    if (sync != hipSuccess) {
      s->result = FH_DEVICE_EXECUTION_FAILED;
      s->error.code = FH_DEVICE_EXECUTION_FAILED;
      s->error.submission = s->serial;
      s->error.value = (uint32_t)sync;
    } else if (s->result == FH_OK) {
      float ms = 0.0f;
      if (hipEventElapsedTime(&ms, s->start, s->end) == hipSuccess)
        s->gpu_ns = (uint64_t)((double)ms * 1e6);
      for (const auto &span : s->spans) {
        float begin_ms = 0.0f, finish_ms = 0.0f;
        if (hipEventElapsedTime(&begin_ms, s->start, span.begin) != hipSuccess ||
            hipEventElapsedTime(&finish_ms, s->start, span.finish) != hipSuccess)
          continue;
        fh_dispatch_timing timing{};
        timing.dispatch = span.first;
        timing.dispatches = span.dispatches;
        timing.op = span.op;
        timing.start_ns = (uint64_t)((double)begin_ms * 1e6);
        timing.end_ns = (uint64_t)((double)finish_ms * 1e6);
        s->timings.push_back(timing);
      }
      for (uint32_t i = 0; i < s->count; ++i) {
        if (!s->host_errors[i].flag) continue;
        s->result = failure_of(s->ops[i], i, s->serial, s->host_errors[i], &s->error);
        break;
      }
    }
    if (b->profiling) {   // the timers of later submissions must have run out before they are read
      (void)hipStreamSynchronize(b->stream);
      drain_profile(b);
    }
  }
  if (error) {
    *error = s->error;
    error->code = s->result;
    error->submission = s->serial;
  }
  return s->result;
}

uint64_t fh_gpu_time_ns(fh_submission *s) { return s ? s->gpu_ns : 0; }

void fh_submission_free(fh_submission *s) {
  if (!s) return;
  fh_backend *b = s->backend;
  std::lock_guard<std::mutex> live(g_live_mutex);
  if (g_live_backends.count(b) == 0) {
    // The device context went with the backend; only the host record remains.
    delete s;
    return;
  }
  {
    std::lock_guard<std::mutex> lock(b->mutex);
    (void)hipSetDevice(b->device);
    if (!s->waited) (void)hipEventSynchronize(s->done);
    b->submissions.erase(s);
    recycle_submission(b, s);
  }
  delete s;
}

fh_status fh_device_info_get(fh_backend *b, fh_device_info *out) {
  if (!b || !out) return FH_INVALID_INPUT;
  memset(out, 0, sizeof(*out));
  snprintf(out->family, sizeof(out->family), "%s", b->props.gcnArchName);
  out->total_memory = b->props.totalGlobalMem;
  out->lds_bytes = b->props.sharedMemPerBlock;
  out->compute_units = (uint32_t)b->props.multiProcessorCount;
  out->wavefront = (uint32_t)b->props.warpSize;
  return FH_OK;
}

fh_status fh_memory_usage(fh_backend *b, uint64_t *bytes) {
  if (!b || !bytes) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  *bytes = b->used_bytes + b->prepared_bytes + b->workspace_bytes + b->accumulator_bytes + b->route_plan_bytes +
           b->attention_plan_bytes + b->lane_scratch_bytes;
  return FH_OK;
}

fh_status fh_set_memory_limit(fh_backend *b, uint64_t bytes) {
  if (!b) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  (void)hipSetDevice(b->device);
  b->memory_limit = bytes;
  if (bytes && b->used_bytes + b->prepared_bytes > bytes) b->evict_prepared();
  return FH_OK;
}

fh_status fh_synchronize(fh_backend *b) {
  if (!b) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  (void)hipSetDevice(b->device);
  if (hipStreamSynchronize(b->stream) != hipSuccess) return FH_DEVICE_EXECUTION_FAILED;
  if (b->profiling) drain_profile(b);
  return FH_OK;
}

fh_status fh_profile_enable(fh_backend *b, int enabled) {
  if (!b) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  (void)hipSetDevice(b->device);
  (void)hipStreamSynchronize(b->stream);
  drain_profile(b);
  b->profiling = enabled < 0 ? 0 : (enabled > 2 ? 2 : enabled);
  return FH_OK;
}

fh_status fh_profile_select(fh_backend *b, uint32_t class_mask) {
  if (!b) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  (void)hipSetDevice(b->device);
  (void)hipStreamSynchronize(b->stream);
  drain_profile(b);
  b->profile_mask = class_mask;
  return FH_OK;
}

fh_status fh_profile_sample(fh_backend *b, uint32_t every) {
  if (!b || every == 0) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  (void)hipSetDevice(b->device);
  (void)hipStreamSynchronize(b->stream);
  drain_profile(b);
  b->profile_every = every;
  for (uint32_t &seen : b->profile_seen) seen = 0;
  return FH_OK;
}

fh_status fh_fusion_enable(fh_backend *b, int enabled) {
  if (!b) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  b->lane_fusion = enabled != 0;
  return FH_OK;
}

fh_status fh_fusion_stats(fh_backend *b, uint64_t *runs, uint64_t *dispatches) {
  if (!b) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  if (runs) *runs = b->fused_runs;
  if (dispatches) *dispatches = b->fused_dispatches;
  return FH_OK;
}

fh_status fh_profile_reset(fh_backend *b) {
  if (!b) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  (void)hipSetDevice(b->device);
  (void)hipStreamSynchronize(b->stream);
  drain_profile(b);
  for (int c = 0; c < FH_KC_COUNT; ++c) {
    b->class_ns[c] = 0;
    b->class_launches[c] = 0;
  }
  return FH_OK;
}

fh_status fh_profile_read(fh_backend *b, uint32_t kernel_class, uint64_t *nanoseconds,
                          uint64_t *launches) {
  if (!b || kernel_class >= FH_KC_COUNT || !nanoseconds || !launches) return FH_INVALID_INPUT;
  std::lock_guard<std::mutex> lock(b->mutex);
  (void)hipSetDevice(b->device);
  (void)hipStreamSynchronize(b->stream);
  drain_profile(b);
  *nanoseconds = b->class_ns[kernel_class];
  *launches = b->class_launches[kernel_class];
  return FH_OK;
}

}  // extern "C"

namespace fh {
char *backend_workspace(fh_backend *backend, uint64_t bytes) { return backend->ensure_workspace(bytes); }
uint64_t backend_workspace_limit(fh_backend *backend) {
  return backend->static_mode ? backend->workspace_bytes : ~0ull;
}
char *backend_route_plan(fh_backend *b, const RoutePlanKey &key, uint64_t bytes, bool *reuse) {
  const RoutePlanKey &have = b->route_plan_key;
  *reuse = b->route_plan_valid && bytes <= b->route_plan_bytes && have.buffer == key.buffer &&
           have.offset == key.offset && have.stride0 == key.stride0 && have.stride1 == key.stride1 &&
           have.rows == key.rows && have.k == key.k && have.experts == key.experts &&
           have.tile == key.tile;
  if (*reuse) return b->route_plan;
  b->route_plan_valid = false;
  if (!b->grow(b->route_plan, b->route_plan_bytes, bytes, 1ull << 20)) return nullptr;
  b->route_plan_key = key;
  b->route_plan_valid = true;
  return b->route_plan;
}
char *backend_attention_plan(fh_backend *b, const AttentionPlanKey &key, uint64_t bytes,
                             bool *reuse) {
  *reuse = b->attention_plan_valid && bytes <= b->attention_plan_bytes &&
           memcmp(&b->attention_plan_key, &key, sizeof(key)) == 0;
  if (*reuse) return b->attention_plan;
  b->attention_plan_valid = false;
  if (!b->grow(b->attention_plan, b->attention_plan_bytes, bytes, 1ull << 20)) return nullptr;
  b->attention_plan_key = key;
  b->attention_plan_valid = true;
  return b->attention_plan;
}
namespace {
bool same_weights(const PreparedKey &l, const PreparedKey &r) {
  for (int i = 0; i < 3; ++i)
    if (l.buffers[i] != r.buffers[i] || l.address[i] != r.address[i]) return false;
  return l.columns == r.columns && l.inner == r.inner;
}
}  // namespace

char *backend_prepared_weights(fh_backend *b, const PreparedKey &key, uint64_t bytes, bool *fresh,
                               int *verdict) {
  *fresh = false;
  *verdict = -1;
  if (b->static_mode) return nullptr;
  for (const auto &e : b->prepared)
    if (same_weights(e.key, key) && (e.bytes == bytes || !e.operand)) {
      *verdict = e.verdict;
      return e.operand;   // null for weights known to be outside the scheme: the verdict is all that is kept
    }
  if (b->prepared_limit == 0) {
    // a quarter of the device's memory unless FORJA_HIP_PREPARED_MB says otherwise (0: keep nothing)
    const char *env = getenv("FORJA_HIP_PREPARED_MB");
    b->prepared_limit = env ? (uint64_t)strtoull(env, nullptr, 10) << 20 : (uint64_t)b->props.totalGlobalMem / 4;
    if (b->prepared_limit == 0) b->prepared_limit = 1;   // asked for nothing: nothing fits
  }
  const uint64_t cost = bytes + fh_backend::kPreparedTail;
  if (b->prepared_bytes + cost > b->prepared_limit) return nullptr;
  if (b->memory_limit && b->used_bytes + b->prepared_bytes + cost > b->memory_limit) return nullptr;
  void *ptr = nullptr;
  if (hipMalloc(&ptr, cost) != hipSuccess) {
    (void)hipGetLastError();   // no room: the workspace serves
    return nullptr;
  }
  b->prepared.push_back({key, (char *)ptr, bytes, -1});
  b->prepared_bytes += cost;
  for (uint64_t watched : key.buffers) ++b->prepared_watch[watched];
  *fresh = true;
  return (char *)ptr;
}

void backend_prepared_verdict(fh_backend *b, const PreparedKey &key) {
  for (auto &e : b->prepared)
    if (same_weights(e.key, key) && e.operand) {
      uint32_t flag = 1;
      if (hipMemcpyAsync(&flag, e.operand + e.bytes, sizeof(flag), hipMemcpyDeviceToHost, b->stream) != hipSuccess ||
          hipStreamSynchronize(b->stream) != hipSuccess)
        return;   // stays unknown: products keep their conditioned second kernel
      e.verdict = flag ? 1 : 0;
      // outside the scheme: the operand is never read again (the stream has just been waited for)
      if (e.verdict == 1) b->free_operand(e);
      return;
    }
}

hipStream_t backend_stream(fh_backend *backend) { return backend->stream; }
uint32_t backend_compute_units(fh_backend *backend) {
  return (uint32_t)backend->props.multiProcessorCount;
}
void backend_profile_begin(fh_backend *backend, uint32_t kernel_class) {
  if (!backend->profiling || kernel_class >= FH_KC_COUNT) return;
  if (!((backend->profile_mask >> kernel_class) & 1u)) return;
  // one launch in `profile_every` of the class is timed (backend_profile_end finds no open timer
  // for the others)
  if (backend->profile_every > 1 && backend->profile_seen[kernel_class]++ % backend->profile_every != 0) return;
  hipEvent_t event = nullptr;
  if (!backend->event_pool.empty()) {
    event = backend->event_pool.back();
    backend->event_pool.pop_back();
  } else if (hipEventCreate(&event) != hipSuccess) {
    return;
  }
  (void)hipEventRecord(event, backend->stream);
  backend->open_timers[kernel_class].push_back(event);
}
void backend_profile_end(fh_backend *backend, uint32_t kernel_class) {
  if (!backend->profiling || kernel_class >= FH_KC_COUNT) return;
  if (backend->open_timers[kernel_class].empty()) return;
  hipEvent_t start = backend->open_timers[kernel_class].back();
  backend->open_timers[kernel_class].pop_back();
  hipEvent_t end = nullptr;
  if (!backend->event_pool.empty()) {
    end = backend->event_pool.back();
    backend->event_pool.pop_back();
  } else if (hipEventCreate(&end) != hipSuccess) {
    backend->event_pool.push_back(start);
    return;
  }
  (void)hipEventRecord(end, backend->stream);
  backend->timed.push_back({start, end, kernel_class});
}
}  // namespace fh
