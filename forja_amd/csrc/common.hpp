// Shared host/device declarations for libforja_hip: strided tensor views, dtype conversion and
// the device error record.  gfx950 only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/forja_hip.h"

namespace fh {

// A tensor as kernels see it: device pointer to element 0 of the allocation plus a Layout in
// element units (crates/forja-core/src/layout.rs).
struct View {
  char *base;
  uint32_t dtype;
  uint32_t rank;
  uint32_t shape[FH_MAX_RANK];
  uint64_t stride[FH_MAX_RANK];
  uint64_t offset;
};

// Data-dependent failure record, one per dispatch of a submission: flag != 0 means the dispatch
// saw an out-of-range index or an unauthenticated page; value is the lowest offender.
struct ErrorSlot {
  uint32_t flag;
  uint32_t value;
};

__host__ __device__ inline uint32_t dtype_size(uint32_t dtype) {
  return (dtype == FH_F16 || dtype == FH_BF16) ? 2u : 4u;
}

#if defined(__HIPCC__)

// A 16-byte load of data the kernel reads once (KV cache rows of a decode step, packed weights of
// a product whose rows fit one tile).  The non-temporal hint keeps such a stream from displacing
// what the caches hold for reuse; a plain read stream over 8 GiB measures 6.1 TB/s on this part
// and 6.8 TB/s with the hint.
__device__ inline uint4 stream_load(const void *address) {
  typedef __attribute__((ext_vector_type(4))) uint32_t words;
  const words v = __builtin_nontemporal_load((const words *)address);
  return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ inline float bf16_to_f32(uint16_t bits) { return __uint_as_float((uint32_t)bits << 16); }

// Round-to-nearest-even, NaN kept quiet: the `half` crate's bf16::from_f32.
__device__ inline uint16_t f32_to_bf16(float value) {
  uint32_t x = __float_as_uint(value);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u);
  x += 0x7fffu + ((x >> 16) & 1u);
  return (uint16_t)(x >> 16);
}

__device__ inline float f16_to_f32(uint16_t bits) {
  _Float16 h;
  __builtin_memcpy(&h, &bits, 2);
  return (float)h;
}

__device__ inline uint16_t f32_to_f16(float value) {
  _Float16 h = (_Float16)value;  // v_cvt_f16_f32: round-to-nearest-even, IEEE overflow/subnormals
  uint16_t bits;
  __builtin_memcpy(&bits, &h, 2);
  return bits;
}

// Element offset of logical row-major index `linear` (element_offsets,
// crates/forja-cpu/src/lib.rs:1736-1745).
__device__ inline uint64_t view_offset(const View &v, uint64_t linear) {
  uint64_t offset = v.offset;
  for (int axis = (int)v.rank - 1; axis >= 0; --axis) {
    uint32_t extent = v.shape[axis];
    offset += (linear % extent) * v.stride[axis];
    linear /= extent;
  }
  return offset;
}

__device__ inline float load_float_at(const View &v, uint64_t element) {
  switch (v.dtype) {
  case FH_F32: return ((const float *)v.base)[element];
  case FH_F16: return f16_to_f32(((const uint16_t *)v.base)[element]);
  default: return bf16_to_f32(((const uint16_t *)v.base)[element]);
  }
}

__device__ inline void store_float_at(const View &v, uint64_t element, float value) {
  switch (v.dtype) {
  case FH_F32: ((float *)v.base)[element] = value; break;
  case FH_F16: ((uint16_t *)v.base)[element] = f32_to_f16(value); break;
  default: ((uint16_t *)v.base)[element] = f32_to_bf16(value); break;
  }
}

__device__ inline uint32_t load_u32_at(const View &v, uint64_t element) {
  return ((const uint32_t *)v.base)[element];
}

// Rounds through the storage dtype, as a store followed by a load would.
__device__ inline float round_to(uint32_t dtype, float value) {
  switch (dtype) {
  case FH_F16: return f16_to_f32(f32_to_f16(value));
  case FH_BF16: return bf16_to_f32(f32_to_bf16(value));
  default: return value;
  }
}

__device__ inline void report_error(ErrorSlot *slot, uint32_t value) {
  atomicMin(&slot->value, value);
  atomicOr(&slot->flag, 1u);
}

// IEEE-754 totalOrder key (f32::total_cmp).
__device__ inline int32_t total_key(float value) {
  int32_t bits = (int32_t)__float_as_uint(value);
  return bits ^ (int32_t)(((uint32_t)(bits >> 31)) >> 1);
}

#endif  // __HIPCC__

}  // namespace fh
