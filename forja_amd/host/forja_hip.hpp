// forja_hip.hpp - C++ host side of the HIP backend, above the C ABI of libforja_hip.so.
//
// It mirrors the surface of `forja_core::Backend` (crates/forja-core/src/backend.rs:650-984) as
// `forja_cpu::CpuBackend` implements it (crates/forja-cpu/src/lib.rs:1335-1517): the same method
// names, argument meaning and error behaviour, so a Rust `impl Backend for HipBackend` is a
// line-by-line transliteration of this file over the same C entry points.  Results are returned
// as `Result<T>` (value or `BackendError`), like the trait's `Result<T, BackendError>`.
//
// There is no CPU fallback: `HipBackend::create` fails when no gfx950 device is visible.
#pragma once

#include <cstdint>
#include <cstring>
#include <string>
#include <utility>
#include <vector>

#include "forja_hip.h"

namespace forja_hip {

enum class DType : uint32_t { F32 = FH_F32, F16 = FH_F16, BF16 = FH_BF16, I32 = FH_I32, U32 = FH_U32 };
inline uint32_t dtype_bytes(DType d) { return (d == DType::F16 || d == DType::BF16) ? 2u : 4u; }

// BackendError (crates/forja-core/src/backend.rs:363-426): a copyable code plus payload.
struct BackendError {
  fh_status code = FH_OK;
  uint32_t dispatch = 0;    // first failing dispatch of the submission
  uint32_t operation = 0;   // fh_op_kind that raised a data-dependent flag
  uint32_t flag = 0;
  uint32_t value = 0;       // lowest offending index / logical page
  bool ok() const { return code == FH_OK; }
};

template <class T>
struct Result {
  T value{};
  BackendError error{};
  bool ok() const { return error.ok(); }
  static Result failure(fh_status code) {
    Result r;
    r.error.code = code;
    return r;
  }
};
struct Unit {};

// Layout (crates/forja-core/src/layout.rs): element-unit strides and offset over a buffer.
struct Layout {
  std::vector<uint32_t> shape;
  std::vector<uint64_t> stride;
  uint64_t offset = 0;

  static Layout contiguous(const std::vector<uint32_t> &shape) {
    Layout l;
    l.shape = shape;
    l.stride.assign(shape.size(), 1);
    for (int axis = (int)shape.size() - 2; axis >= 0; --axis)
      l.stride[axis] = l.stride[axis + 1] * shape[axis + 1];
    return l;
  }
  uint64_t elements() const {
    uint64_t n = 1;
    for (uint32_t extent : shape) n *= extent;
    return n;
  }
  bool is_contiguous() const {
    uint64_t expected = 1;
    for (int axis = (int)shape.size() - 1; axis >= 0; --axis) {
      if (shape[axis] != 1 && stride[axis] != expected) return false;
      expected *= shape[axis];
    }
    return true;
  }
};

// ViewOp (crates/forja-core/src/backend.rs: `ViewOp::{Slice, Permute, Broadcast, Reshape}`).
struct SliceSpec {
  uint32_t start, length, step;
};

// Tensor = (BufferId, Layout, writable), crates/forja-core/src/ops.rs:62-160.
struct Tensor {
  fh_buffer buffer = 0;
  DType dtype = DType::F32;
  Layout layout;
  bool writable = true;

  // Tensor::narrow: the sub-range [start, start+length) of one axis.
  Tensor narrow(uint32_t axis, uint32_t start, uint32_t length) const {
    Tensor t = *this;
    t.layout.offset += (uint64_t)start * layout.stride[axis];
    t.layout.shape[axis] = length;
    return t;
  }
  Tensor slice(const std::vector<SliceSpec> &specs) const {
    Tensor t = *this;
    for (size_t axis = 0; axis < specs.size(); ++axis) {
      t.layout.offset += (uint64_t)specs[axis].start * layout.stride[axis];
      t.layout.shape[axis] = specs[axis].length;
      t.layout.stride[axis] = layout.stride[axis] * specs[axis].step;
    }
    return t;
  }
  Tensor permute(const std::vector<uint32_t> &axes) const {
    Tensor t = *this;
    for (size_t i = 0; i < axes.size(); ++i) {
      t.layout.shape[i] = layout.shape[axes[i]];
      t.layout.stride[i] = layout.stride[axes[i]];
    }
    return t;
  }
  Tensor broadcast(const std::vector<uint32_t> &shape) const {
    Tensor t = *this;
    size_t lead = shape.size() - layout.shape.size();
    t.layout.shape = shape;
    t.layout.stride.assign(shape.size(), 0);
    for (size_t axis = 0; axis < layout.shape.size(); ++axis)
      t.layout.stride[lead + axis] = layout.shape[axis] == 1 ? 0 : layout.stride[axis];
    t.writable = false;
    return t;
  }
  fh_tensor raw() const {
    fh_tensor r{};
    r.buffer = buffer;
    r.dtype = (uint32_t)dtype;
    r.rank = (uint32_t)layout.shape.size();
    for (size_t axis = 0; axis < layout.shape.size(); ++axis) {
      r.shape[axis] = layout.shape[axis];
      r.stride[axis] = layout.stride[axis];
    }
    r.offset = layout.offset;
    return r;
  }
};

// Op (crates/forja-core/src/ops.rs:163-302): constructors fill the C dispatch record.
struct Op {
  fh_dispatch record{};
  static Op of(fh_op_kind kind) {
    Op op;
    op.record.op = kind;
    return op;
  }
  static Op copy() { return of(FH_OP_COPY); }
  static Op argmax() { return of(FH_OP_ARGMAX); }
  static Op matmul() { return of(FH_OP_MATMUL); }
  static Op rms_norm(float eps) {
    Op op = of(FH_OP_RMS_NORM);
    op.record.eps = eps;
    return op;
  }
  static Op rope(float theta) {
    Op op = of(FH_OP_ROPE);
    op.record.theta = theta;
    return op;
  }
  // Op::Sample / Op::SampleMasked: the position travels in `start`; the Metal tuning attributes
  // (chunk_width, fast_top_k, ...) stay on the host side of the boundary.
  static Op sample(uint32_t position) {
    Op op = of(FH_OP_SAMPLE);
    op.record.start = position;
    return op;
  }
  static Op sample_masked(uint32_t position) {
    Op op = of(FH_OP_SAMPLE_MASKED);
    op.record.start = position;
    return op;
  }
  static Op top_k(uint32_t k, bool normalize) {
    Op op = of(FH_OP_TOP_K);
    op.record.k = k;
    op.record.normalize = normalize;
    return op;
  }
  static Op quant_embed(uint32_t bits, uint32_t group_size) {
    Op op = of(FH_OP_QUANT_EMBED);
    op.record.bits = bits;
    op.record.group_size = group_size;
    return op;
  }
  static Op quant_matmul(uint32_t bits, uint32_t group_size) {
    Op op = of(FH_OP_QUANT_MATMUL);
    op.record.bits = bits;
    op.record.group_size = group_size;
    return op;
  }
  static Op gather_quant_matmul(uint32_t bits, uint32_t group_size) {
    Op op = of(FH_OP_GATHER_QUANT_MATMUL);
    op.record.bits = bits;
    op.record.group_size = group_size;
    return op;
  }
  static Op paged_copy(bool out_of_pages, uint32_t start, uint32_t page_tokens) {
    Op op = of(FH_OP_PAGED_COPY);
    op.record.direction = out_of_pages;
    op.record.start = start;
    op.record.page_tokens = page_tokens;
    return op;
  }
  static Op paged_sdpa(float scale, bool causal, uint32_t q_start, uint32_t key_length,
                       uint32_t page_tokens) {
    Op op = of(FH_OP_PAGED_SDPA);
    op.record.scale = scale;
    op.record.causal = causal;
    op.record.q_start = q_start;
    op.record.key_length = key_length;
    op.record.page_tokens = page_tokens;
    return op;
  }
  static Op paged_sdpa_append(float scale, uint32_t q_start, uint32_t page_tokens) {
    Op op = of(FH_OP_PAGED_SDPA_APPEND);
    op.record.scale = scale;
    op.record.q_start = q_start;
    op.record.page_tokens = page_tokens;
    return op;
  }
  // one_row_per_lane: the recorder's promise of a decode batch, checked when the dispatch runs
  static Op paged_attention_ragged(float scale, uint32_t page_tokens, bool one_row_per_lane = false) {
    Op op = of(FH_OP_PAGED_ATTENTION_RAGGED);
    op.record.scale = scale;
    op.record.page_tokens = page_tokens;
    op.record.k = one_row_per_lane ? 1 : 0;
    return op;
  }
};

// CommandList (crates/forja-core/src/ops.rs:445-620): dispatches in recording order.
class CommandList {
 public:
  void dispatch(const Op &op, const std::vector<Tensor> &inputs, const std::vector<Tensor> &outputs) {
    fh_dispatch d = op.record;
    fill(d, inputs, outputs);
    dispatches_.push_back(d);
  }
  // Op::Program through a prepared handle.
  void dispatch_kernel(fh_program program, const std::vector<Tensor> &inputs,
                       const std::vector<Tensor> &outputs) {
    fh_dispatch d{};
    d.op = FH_OP_PROGRAM;
    d.program = program;
    fill(d, inputs, outputs);
    dispatches_.push_back(d);
  }
  // A matmul-family op with a fused epilogue program; `extras` follow the primitive inputs.
  void dispatch_epilogue(const Op &op, std::vector<Tensor> inputs, const Tensor &output,
                         fh_program epilogue, const std::vector<Tensor> &extras,
                         uint32_t accumulator_count = 1) {
    fh_dispatch d = op.record;
    d.epilogue = epilogue;
    d.accumulator_count = accumulator_count;
    d.n_extras = (uint32_t)extras.size();
    inputs.insert(inputs.end(), extras.begin(), extras.end());
    fill(d, inputs, {output});
    dispatches_.push_back(d);
  }
  const std::vector<fh_dispatch> &dispatches() const { return dispatches_; }
  bool empty() const { return dispatches_.empty(); }

 private:
  static void fill(fh_dispatch &d, const std::vector<Tensor> &inputs, const std::vector<Tensor> &outputs) {
    d.n_inputs = (uint32_t)inputs.size();
    d.n_outputs = (uint32_t)outputs.size();
    for (size_t i = 0; i < inputs.size() && i < FH_MAX_INPUTS; ++i) d.inputs[i] = inputs[i].raw();
    for (size_t i = 0; i < outputs.size() && i < FH_MAX_OUTPUTS; ++i) d.outputs[i] = outputs[i].raw();
  }
  std::vector<fh_dispatch> dispatches_;
};

// Submission (crates/forja-core/src/backend.rs:609-647).
class Submission {
 public:
  Submission() = default;
  explicit Submission(fh_submission *raw) : raw_(raw) {}
  Submission(Submission &&other) noexcept : raw_(other.raw_) { other.raw_ = nullptr; }
  Submission &operator=(Submission &&other) noexcept {
    if (this != &other) {
      reset();
      raw_ = other.raw_;
      other.raw_ = nullptr;
    }
    return *this;
  }
  Submission(const Submission &) = delete;
  Submission &operator=(const Submission &) = delete;
  ~Submission() { reset(); }

  // Blocks until the work has finished; a data-dependent device flag surfaces here, as it does
  // from `Submission::wait` in the reference.
  Result<Unit> wait() { return wait_timeout(0); }
  Result<Unit> wait_timeout(uint64_t nanoseconds) {
    Result<Unit> r;
    if (!raw_) return r;
    fh_error e{};
    fh_status status = fh_wait(raw_, nanoseconds, &e);
    r.error.code = status;
    r.error.dispatch = e.dispatch;
    r.error.operation = e.operation;
    r.error.flag = e.flag;
    r.error.value = e.value;
    return r;
  }
  uint64_t gpu_time_ns() const { return raw_ ? fh_gpu_time_ns(raw_) : 0; }
  // Submission::profile: the per-dispatch device timeline of a submission made by
  // submit_profiled, once it has been waited for (empty otherwise).
  std::vector<fh_dispatch_timing> profile() const {
    std::vector<fh_dispatch_timing> timings;
    uint32_t n = 0;
    if (!raw_ || fh_submission_profile(raw_, nullptr, 0, &n) != FH_OK || n == 0) return timings;
    timings.resize(n);
    if (fh_submission_profile(raw_, timings.data(), n, &n) != FH_OK) timings.clear();
    return timings;
  }

 private:
  void reset() {
    if (raw_) fh_submission_free(raw_);
    raw_ = nullptr;
  }
  fh_submission *raw_ = nullptr;
};

struct Inst {
  uint32_t kind, op, a, b, c;
};
struct Program {
  uint32_t kind = 0;                 // 0 map, 1 row
  std::vector<Inst> insts;
  std::vector<std::pair<uint32_t, uint32_t>> outputs;  // (output slot, value id)
};

class HipBackend {
 public:
  static Result<HipBackend *> create(int device = 0) {
    Result<HipBackend *> r;
    fh_backend *raw = nullptr;
    r.error.code = fh_create(device, &raw);
    if (r.ok()) r.value = new HipBackend(raw);
    return r;
  }
  ~HipBackend() { fh_destroy(raw_); }
  HipBackend(const HipBackend &) = delete;
  HipBackend &operator=(const HipBackend &) = delete;

  // Backend::alloc: zero-initialised contiguous tensor.
  Result<Tensor> alloc(DType dtype, const std::vector<uint32_t> &shape) {
    Result<Tensor> r;
    if (shape.size() > FH_MAX_RANK) return Result<Tensor>::failure(FH_INVALID_INPUT);
    Layout layout = Layout::contiguous(shape);
    uint64_t bytes = layout.elements() * dtype_bytes(dtype);
    r.error.code = fh_alloc(raw_, bytes, &r.value.buffer);
    r.value.dtype = dtype;
    r.value.layout = layout;
    return r;
  }
  // Backend::import_readonly: a read-only copy of host bytes (weights).
  Result<Tensor> import_readonly(DType dtype, const std::vector<uint32_t> &shape, const void *bytes,
                                 uint64_t len) {
    Result<Tensor> r;
    Layout layout = Layout::contiguous(shape);
    if (layout.elements() * dtype_bytes(dtype) != len) return Result<Tensor>::failure(FH_INVALID_INPUT);
    r.error.code = fh_import(raw_, bytes, len, &r.value.buffer);
    r.value.dtype = dtype;
    r.value.layout = layout;
    r.value.writable = false;
    return r;
  }
  // Backend::write: contiguous + writable + exact length, else InvalidInput.
  Result<Unit> write(const Tensor &tensor, const void *bytes, uint64_t len) {
    if (!tensor.writable || !tensor.layout.is_contiguous() ||
        len != tensor.layout.elements() * dtype_bytes(tensor.dtype))
      return Result<Unit>::failure(FH_INVALID_INPUT);
    Result<Unit> r;
    r.error.code = fh_write(raw_, tensor.buffer, tensor.layout.offset * dtype_bytes(tensor.dtype), bytes, len);
    return r;
  }
  // Backend::read: the view's logical row-major bytes.
  Result<std::vector<uint8_t>> read(const Tensor &tensor) {
    Result<std::vector<uint8_t>> r;
    r.value.resize(tensor.layout.elements() * dtype_bytes(tensor.dtype));
    fh_tensor raw = tensor.raw();
    r.error.code = fh_read_tensor(raw_, &raw, r.value.data(), r.value.size());
    return r;
  }
  Result<std::vector<uint8_t>> read_buffer_range(fh_buffer buffer, uint64_t byte_offset, uint64_t len) {
    Result<std::vector<uint8_t>> r;
    r.value.resize(len);
    r.error.code = fh_read(raw_, buffer, byte_offset, r.value.data(), len);
    return r;
  }
  Result<Unit> release(const Tensor &tensor) {
    Result<Unit> r;
    r.error.code = fh_release(raw_, tensor.buffer);
    return r;
  }
  Result<fh_program> prepare_program(const Program &program) {
    Result<fh_program> r;
    std::vector<fh_inst> insts(program.insts.size());
    for (size_t i = 0; i < insts.size(); ++i)
      insts[i] = fh_inst{program.insts[i].kind, program.insts[i].op, program.insts[i].a,
                         program.insts[i].b, program.insts[i].c};
    std::vector<uint32_t> pairs;
    for (auto &pair : program.outputs) {
      pairs.push_back(pair.first);
      pairs.push_back(pair.second);
    }
    r.error.code = fh_prepare_program(raw_, program.kind, insts.data(), (uint32_t)insts.size(),
                                      pairs.data(), (uint32_t)program.outputs.size(), &r.value);
    return r;
  }
  // Backend::submit: validates, enqueues, returns without waiting.
  Result<Submission> submit(const CommandList &commands) {
    Result<Submission> r;
    fh_submission *raw = nullptr;
    r.error.code = fh_submit(raw_, commands.dispatches().data(), (uint32_t)commands.dispatches().size(), &raw);
    if (r.ok()) r.value = Submission(raw);
    return r;
  }
  // Backend::submit_profiled_retained: submit with a device timer around every dispatch.
  Result<Submission> submit_profiled(const CommandList &commands) {
    Result<Submission> r;
    fh_submission *raw = nullptr;
    r.error.code = fh_submit_profiled(raw_, commands.dispatches().data(), (uint32_t)commands.dispatches().size(), &raw);
    if (r.ok()) r.value = Submission(raw);
    return r;
  }
  Result<fh_device_info> device_info() {
    Result<fh_device_info> r;
    r.error.code = fh_device_info_get(raw_, &r.value);
    return r;
  }
  Result<uint64_t> memory_usage() {
    Result<uint64_t> r;
    r.error.code = fh_memory_usage(raw_, &r.value);
    return r;
  }
  // Backend::set_memory_limit: quota over allocations plus the operands the library keeps.
  Result<Unit> set_memory_limit(uint64_t bytes) {
    Result<Unit> r;
    r.error.code = fh_set_memory_limit(raw_, bytes);
    return r;
  }
  Result<Unit> synchronize() {
    Result<Unit> r;
    r.error.code = fh_synchronize(raw_);
    return r;
  }
  fh_backend *raw() { return raw_; }

 private:
  explicit HipBackend(fh_backend *raw) : raw_(raw) {}
  fh_backend *raw_;
};

}  // namespace forja_hip
