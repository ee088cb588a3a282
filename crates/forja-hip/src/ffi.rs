//! Raw bindings of include/forja_hip.h, declaration for declaration.
#![allow(non_camel_case_types, missing_docs, clippy::missing_safety_doc)]

use std::os::raw::{c_char, c_int, c_void};

pub const FH_MAX_RANK: usize = 8;
pub const FH_MAX_INPUTS: usize = 12;
pub const FH_MAX_OUTPUTS: usize = 4;

// fh_status: the discriminants of `forja_core::BackendError`, in declaration order.
pub const FH_OK: u32 = 0;
pub const FH_QUOTA_EXCEEDED: u32 = 1;
pub const FH_ALLOCATION_FAILED: u32 = 2;
pub const FH_INVALID_DEVICE_WORKING_SET: u32 = 3;
pub const FH_EXECUTION_FAILED: u32 = 4;
pub const FH_DEVICE_EXECUTION_FAILED: u32 = 5;
pub const FH_DEVICE_ERROR_FLAG: u32 = 6;
pub const FH_GPU_PREDICTION_EXCEEDED: u32 = 7;
pub const FH_IMPOSSIBLE_RATE: u32 = 8;
pub const FH_TIMEOUT: u32 = 9;
pub const FH_INVALID_INPUT: u32 = 10;
pub const FH_UNSUPPORTED_OPERATION: u32 = 11;
pub const FH_INDEX_OUT_OF_RANGE: u32 = 12;

// fh_dtype
pub const FH_F32: u32 = 0;
pub const FH_F16: u32 = 1;
pub const FH_BF16: u32 = 2;
pub const FH_I32: u32 = 3;
pub const FH_U32: u32 = 4;

// fh_op_kind
pub const FH_OP_PROGRAM: u32 = 1;
pub const FH_OP_COPY: u32 = 2;
pub const FH_OP_PAGED_COPY: u32 = 3;
pub const FH_OP_RMS_NORM: u32 = 4;
pub const FH_OP_ARGMAX: u32 = 5;
pub const FH_OP_TOP_K: u32 = 6;
pub const FH_OP_ROPE: u32 = 7;
pub const FH_OP_QUANT_EMBED: u32 = 8;
pub const FH_OP_MATMUL: u32 = 9;
pub const FH_OP_QUANT_MATMUL: u32 = 10;
pub const FH_OP_GATHER_QUANT_MATMUL: u32 = 11;
pub const FH_OP_PAGED_SDPA_APPEND: u32 = 12;
pub const FH_OP_PAGED_SDPA: u32 = 13;
pub const FH_OP_SAMPLE: u32 = 14;
pub const FH_OP_SAMPLE_MASKED: u32 = 15;
pub const FH_OP_PAGED_ATTENTION_RAGGED: u32 = 32;
pub const FH_OP_ROUTE_PACK: u32 = 33;
pub const FH_OP_FILL_SEEDED: u32 = 34;

#[repr(C)]
pub struct fh_backend {
    _private: [u8; 0],
}
#[repr(C)]
pub struct fh_submission {
    _private: [u8; 0],
}
pub type fh_buffer = u64;
pub type fh_program = u64;

#[repr(C)]
#[derive(Clone, Copy, Default)]
pub struct fh_tensor {
    pub buffer: fh_buffer,
    pub dtype: u32,
    pub rank: u32,
    pub shape: [u32; FH_MAX_RANK],
    pub stride: [u64; FH_MAX_RANK],
    pub offset: u64,
}

#[repr(C)]
#[derive(Clone, Copy, Default)]
pub struct fh_inst {
    pub kind: u32,
    pub op: u32,
    pub a: u32,
    pub b: u32,
    pub c: u32,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct fh_dispatch {
    pub op: u32,
    pub scale: f32,
    pub eps: f32,
    pub theta: f32,
    pub bits: u32,
    pub group_size: u32,
    pub k: u32,
    pub normalize: u32,
    pub causal: u32,
    pub q_start: u32,
    pub key_length: u32,
    pub page_tokens: u32,
    pub direction: u32,
    pub start: u32,
    pub n_inputs: u32,
    pub n_outputs: u32,
    pub program: fh_program,
    pub epilogue: fh_program,
    pub accumulator_count: u32,
    pub n_extras: u32,
    pub inputs: [fh_tensor; FH_MAX_INPUTS],
    pub outputs: [fh_tensor; FH_MAX_OUTPUTS],
}

impl Default for fh_dispatch {
    fn default() -> Self {
        // Every field is an integer, a float or an array of them: all-zero is a valid value.
        unsafe { std::mem::zeroed() }
    }
}

#[repr(C)]
#[derive(Clone, Copy, Default)]
pub struct fh_error {
    pub code: u32,
    pub dispatch: u32,
    pub submission: u64,
    pub operation: u32,
    pub flag: u32,
    pub value: u32,
    pub reserved: u32,
}

#[repr(C)]
pub struct fh_device_info {
    pub family: [c_char; 64],
    pub total_memory: u64,
    pub lds_bytes: u64,
    pub compute_units: u32,
    pub wavefront: u32,
}

unsafe /// `fh_dispatch_timing`: device time from the start of a submission to the start and end of one
/// executed dispatch (or group of dispatches executed together).
#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct fh_dispatch_timing {
    pub dispatch: u32,
    pub dispatches: u32,
    pub op: u32,
    pub reserved: u32,
    pub start_ns: u64,
    pub end_ns: u64,
}

extern "C" {
    pub fn fh_create(device: c_int, out: *mut *mut fh_backend) -> u32;
    pub fn fh_destroy(backend: *mut fh_backend);
    pub fn fh_alloc(backend: *mut fh_backend, bytes: u64, out: *mut fh_buffer) -> u32;
    pub fn fh_release(backend: *mut fh_backend, buffer: fh_buffer) -> u32;
    pub fn fh_import(backend: *mut fh_backend, bytes: *const c_void, len: u64, out: *mut fh_buffer) -> u32;
    pub fn fh_write(backend: *mut fh_backend, buffer: fh_buffer, byte_offset: u64, bytes: *const c_void, len: u64) -> u32;
    pub fn fh_read(backend: *mut fh_backend, buffer: fh_buffer, byte_offset: u64, bytes: *mut c_void, len: u64) -> u32;
    pub fn fh_read_tensor(backend: *mut fh_backend, tensor: *const fh_tensor, bytes: *mut c_void, len: u64) -> u32;
    pub fn fh_prepare_program(
        backend: *mut fh_backend,
        kind: u32,
        insts: *const fh_inst,
        n_insts: u32,
        outputs: *const u32,
        n_pairs: u32,
        out: *mut fh_program,
    ) -> u32;
    pub fn fh_release_program(backend: *mut fh_backend, program: fh_program) -> u32;
    pub fn fh_submit(backend: *mut fh_backend, dispatches: *const fh_dispatch, count: u32, out: *mut *mut fh_submission) -> u32;
    pub fn fh_submit_static(backend: *mut fh_backend, dispatches: *const fh_dispatch, count: u32, error: *mut fh_error) -> u32;
    pub fn fh_wait(submission: *mut fh_submission, timeout_ns: u64, error: *mut fh_error) -> u32;
    pub fn fh_gpu_time_ns(submission: *mut fh_submission) -> u64;
    pub fn fh_submission_free(submission: *mut fh_submission);
    pub fn fh_device_info_get(backend: *mut fh_backend, out: *mut fh_device_info) -> u32;
    pub fn fh_memory_usage(backend: *mut fh_backend, bytes: *mut u64) -> u32;
    pub fn fh_set_memory_limit(backend: *mut fh_backend, bytes: u64) -> u32;
    pub fn fh_submit_profiled(backend: *mut fh_backend, dispatches: *const fh_dispatch, count: u32, out: *mut *mut fh_submission) -> u32;
    pub fn fh_submission_profile(submission: *mut fh_submission, out: *mut fh_dispatch_timing, capacity: u32, n: *mut u32) -> u32;
    pub fn fh_synchronize(backend: *mut fh_backend) -> u32;
    pub fn fh_profile_enable(backend: *mut fh_backend, enabled: c_int) -> u32;
    pub fn fh_profile_select(backend: *mut fh_backend, class_mask: u32) -> u32;
    pub fn fh_profile_sample(backend: *mut fh_backend, every: u32) -> u32;
    pub fn fh_profile_reset(backend: *mut fh_backend) -> u32;
    pub fn fh_profile_read(backend: *mut fh_backend, kernel_class: u32, nanoseconds: *mut u64, launches: *mut u64) -> u32;
    pub fn fh_fusion_enable(backend: *mut fh_backend, enabled: c_int) -> u32;
    pub fn fh_fusion_stats(backend: *mut fh_backend, runs: *mut u64, dispatches: *mut u64) -> u32;
    pub fn fh_version() -> *const c_char;
}
