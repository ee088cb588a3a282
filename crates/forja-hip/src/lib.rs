//! `HipBackend`: forja's execution backend for AMD MI355X (gfx950).
//!
//! Everything that touches the device lives in libforja_hip.so (hand-written HIP kernels behind
//! the C ABI of include/forja_hip.h).  This crate is the thin trusted shim that lets the host use
//! it through `forja_core::Backend`, method for method the way `forja-cpu` implements the trait
//! (crates/forja-cpu/src/lib.rs:1335-1517): allocation identities and view validation stay in
//! `AllocationRegistry`, every dispatch is lowered to an `fh_dispatch`, and data-dependent
//! failures come back as the `BackendError` variants the Metal backend uses.
//!
//! Not compiled in the build image of the HIP library (it has no Rust toolchain); the C++ mirror
//! forja_amd/host/forja_hip.hpp is the same shim, compiled and run against the device.
#![allow(unsafe_code)]

pub mod ffi;

use std::collections::HashMap;
use std::ops::Range;
use std::ptr::NonNull;
use std::sync::{Arc, Mutex};
use std::time::Duration;

use forja_core::{
    AllocationRegistry, Backend, BackendError, BinOp, BufferId, CommandList, CompletionResource,
    DType, DeviceInfo, Dispatch, DispatchProfile, Inst, KernelCost, KernelSignature, Layout,
    MemoryUsage, Op, PagedCopyDirection, ProfileTensor, ProgramKind, ReadonlyImport, RedOp,
    Submission, SubmissionProfile, Tensor, UnOp, ValidatedProgram, ValueType, ViewOp,
};
use forja_mmap::MappedRegion;

use ffi::{fh_dispatch, fh_error, fh_inst, fh_tensor};

/// Owner of the C-side backend object; shared by the backend, its programs and its submissions
/// so that none of them outlives the device context it refers to.
struct RawBackend(NonNull<ffi::fh_backend>);

// libforja_hip serialises internally (one mutex per backend); every entry point may be called
// from any thread.
unsafe impl Send for RawBackend {}
unsafe impl Sync for RawBackend {}

impl RawBackend {
    fn ptr(&self) -> *mut ffi::fh_backend {
        self.0.as_ptr()
    }
}

impl Drop for RawBackend {
    fn drop(&mut self) {
        unsafe { ffi::fh_destroy(self.ptr()) }
    }
}

/// Device storage behind one allocation identity.
#[derive(Debug)]
struct HipBuffer {
    handle: ffi::fh_buffer,
    raw: Arc<RawBackend>,
}

impl std::fmt::Debug for RawBackend {
    fn fmt(&self, formatter: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        formatter.write_str("RawBackend")
    }
}

impl Drop for HipBuffer {
    fn drop(&mut self) {
        // Removing the registry entry releases the device allocation and with it every view.
        let _ = unsafe { ffi::fh_release(self.raw.ptr(), self.handle) };
    }
}

/// A scalar program the library has validated and keeps ready (`Backend::ProgramHandle`).
#[derive(Debug)]
pub struct HipProgram {
    handle: ffi::fh_program,
    raw: Arc<RawBackend>,
}

impl Drop for HipProgram {
    fn drop(&mut self) {
        let _ = unsafe { ffi::fh_release_program(self.raw.ptr(), self.handle) };
    }
}

/// The MI355X backend.
pub struct HipBackend {
    raw: Arc<RawBackend>,
    buffers: Mutex<AllocationRegistry<HipBuffer>>,
    /// Epilogue programs carry no backend handle (`PreparedEpilogue`,
    /// crates/forja-core/src/program.rs:317-345): they are prepared on first use, by content.
    epilogues: Mutex<HashMap<[u8; 32], Arc<HipProgram>>>,
}

impl std::fmt::Debug for HipBackend {
    fn fmt(&self, formatter: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        formatter.debug_struct("HipBackend").finish_non_exhaustive()
    }
}

/// Operation names reported in `BackendError::DeviceErrorFlag`, by `fh_op_kind`; the names the
/// Metal backend reports (crates/forja-metal/tests/paged.rs:239-277,
/// crates/forja-metal/tests/gather_quant_matmul.rs:742-764).
fn operation_name(kind: u32) -> &'static str {
    match kind {
        ffi::FH_OP_PROGRAM => "program",
        ffi::FH_OP_COPY => "copy",
        ffi::FH_OP_PAGED_COPY => "paged-copy",
        ffi::FH_OP_RMS_NORM => "rms-norm",
        ffi::FH_OP_ARGMAX => "argmax",
        ffi::FH_OP_TOP_K => "top-k",
        ffi::FH_OP_ROPE => "rope",
        ffi::FH_OP_QUANT_EMBED => "quant-embed",
        ffi::FH_OP_MATMUL => "matmul",
        ffi::FH_OP_QUANT_MATMUL => "quant-matmul",
        ffi::FH_OP_GATHER_QUANT_MATMUL => "gather-quant-matmul",
        ffi::FH_OP_PAGED_SDPA_APPEND => "paged-sdpa-append",
        ffi::FH_OP_PAGED_SDPA => "paged-sdpa",
        ffi::FH_OP_SAMPLE => "sample",
        ffi::FH_OP_SAMPLE_MASKED => "sample-masked",
        _ => "unknown",
    }
}

/// `fh_status` (+ the error record of a wait) as `BackendError`
/// (crates/forja-core/src/backend.rs:363-426).
fn backend_error(status: u32, error: &fh_error) -> BackendError {
    match status {
        ffi::FH_QUOTA_EXCEEDED => BackendError::QuotaExceeded,
        ffi::FH_ALLOCATION_FAILED => BackendError::AllocationFailed,
        ffi::FH_EXECUTION_FAILED => BackendError::ExecutionFailed,
        ffi::FH_DEVICE_EXECUTION_FAILED => BackendError::DeviceExecutionFailed {
            submission: error.submission,
            code: i64::from(error.value),
        },
        ffi::FH_DEVICE_ERROR_FLAG => BackendError::DeviceErrorFlag {
            submission: error.submission,
            dispatch: error.dispatch,
            operation: operation_name(error.operation),
            flag: error.flag,
            value: error.value,
        },
        ffi::FH_TIMEOUT => BackendError::Timeout,
        ffi::FH_UNSUPPORTED_OPERATION => BackendError::UnsupportedOperation,
        ffi::FH_INDEX_OUT_OF_RANGE => BackendError::IndexOutOfRange { index: error.value },
        // FH_INVALID_DEVICE_WORKING_SET, FH_GPU_PREDICTION_EXCEEDED and FH_IMPOSSIBLE_RATE belong
        // to host-side admission; the library never returns them.
        _ => BackendError::InvalidInput,
    }
}

fn check(status: u32) -> Result<(), BackendError> {
    if status == ffi::FH_OK {
        Ok(())
    } else {
        Err(backend_error(status, &fh_error::default()))
    }
}

const fn dtype_code(dtype: DType) -> u32 {
    match dtype {
        DType::F32 => ffi::FH_F32,
        DType::F16 => ffi::FH_F16,
        DType::BF16 => ffi::FH_BF16,
        DType::I32 => ffi::FH_I32,
        DType::U32 => ffi::FH_U32,
    }
}

/// One Program IR instruction in the C ABI's encoding (wit/compute.wit:75-141 order).
fn encode_inst(inst: Inst) -> fh_inst {
    let (kind, op, a, b, c) = match inst {
        Inst::Input(slot) => (0, 0, slot, 0, 0),
        Inst::Const(value) => (1, 0, value.to_bits(), 0, 0),
        Inst::Index(axis) => (2, u32::from(axis), 0, 0, 0),
        Inst::Extent(axis) => (3, u32::from(axis), 0, 0, 0),
        Inst::Unary(op, value) => (4, unop_code(op), value, 0, 0),
        Inst::Binary(op, left, right) => (5, binop_code(op), left, right, 0),
        Inst::Select(condition, accepted, rejected) => (6, 0, condition, accepted, rejected),
        Inst::Cast(to, value) => (7, value_type_code(to), value, 0, 0),
        Inst::Reduce(op, value) => (8, redop_code(op), value, 0, 0),
    };
    fh_inst { kind, op, a, b, c }
}

const fn unop_code(op: UnOp) -> u32 {
    match op {
        UnOp::Neg => 0,
        UnOp::Abs => 1,
        UnOp::Exp => 2,
        UnOp::Log => 3,
        UnOp::Sqrt => 4,
        UnOp::Rsqrt => 5,
        UnOp::Sin => 6,
        UnOp::Cos => 7,
        UnOp::Tanh => 8,
        UnOp::Sigmoid => 9,
        UnOp::Recip => 10,
        UnOp::Floor => 11,
        UnOp::Log1p => 12,
        UnOp::ExpRounded => 13,
    }
}

const fn binop_code(op: BinOp) -> u32 {
    match op {
        BinOp::Add => 0,
        BinOp::Sub => 1,
        BinOp::Mul => 2,
        BinOp::Div => 3,
        BinOp::Min => 4,
        BinOp::Max => 5,
        BinOp::Pow => 6,
        BinOp::Lt => 7,
        BinOp::Le => 8,
        BinOp::Eq => 9,
        BinOp::Ne => 10,
        BinOp::Ge => 11,
        BinOp::Gt => 12,
    }
}

const fn redop_code(op: RedOp) -> u32 {
    match op {
        RedOp::Sum => 0,
        RedOp::Max => 1,
        RedOp::Min => 2,
    }
}

const fn value_type_code(value: ValueType) -> u32 {
    match value {
        ValueType::F32 => 0,
        ValueType::U32 => 1,
        ValueType::Bool => 2,
    }
}

impl HipBackend {
    /// Opens device `device` (an index among the visible gfx950 devices).
    ///
    /// # Errors
    ///
    /// Returns a device execution failure when no such device is visible: there is no CPU
    /// fallback.
    pub fn new(device: i32) -> Result<Self, BackendError> {
        let mut raw = std::ptr::null_mut();
        check(unsafe { ffi::fh_create(device, &mut raw) })?;
        let raw = NonNull::new(raw).ok_or(BackendError::ExecutionFailed)?;
        Ok(Self {
            raw: Arc::new(RawBackend(raw)),
            buffers: Mutex::new(AllocationRegistry::new()),
            epilogues: Mutex::new(HashMap::new()),
        })
    }

    fn registry(
        &self,
    ) -> Result<std::sync::MutexGuard<'_, AllocationRegistry<HipBuffer>>, BackendError> {
        self.buffers.lock().map_err(|_| BackendError::ExecutionFailed)
    }

    /// A tensor as the C ABI names it, after the registry has vouched for its identity.
    fn lower_tensor(
        registry: &AllocationRegistry<HipBuffer>,
        tensor: &Tensor,
    ) -> Result<fh_tensor, BackendError> {
        let storage = registry.get(tensor)?;
        let layout = tensor.layout();
        let rank = layout.shape().len();
        if rank > ffi::FH_MAX_RANK {
            return Err(BackendError::InvalidInput);
        }
        let mut lowered = fh_tensor {
            buffer: storage.handle,
            dtype: dtype_code(layout.dtype()),
            rank: u32::try_from(rank).map_err(|_| BackendError::InvalidInput)?,
            offset: layout.offset(),
            ..fh_tensor::default()
        };
        lowered.shape[..rank].copy_from_slice(layout.shape());
        lowered.stride[..rank].copy_from_slice(layout.strides());
        Ok(lowered)
    }

    fn prepare_raw(&self, program: &ValidatedProgram) -> Result<HipProgram, BackendError> {
        let source = program.program();
        let insts: Vec<fh_inst> = source.insts.iter().copied().map(encode_inst).collect();
        let pairs: Vec<u32> = source.outputs.iter().flat_map(|&(slot, value)| [slot, value]).collect();
        let kind = match source.kind {
            ProgramKind::Map => 0,
            ProgramKind::Row => 1,
        };
        let mut handle = 0;
        check(unsafe {
            ffi::fh_prepare_program(
                self.raw.ptr(),
                kind,
                insts.as_ptr(),
                u32::try_from(insts.len()).map_err(|_| BackendError::InvalidInput)?,
                pairs.as_ptr(),
                u32::try_from(source.outputs.len()).map_err(|_| BackendError::InvalidInput)?,
                &mut handle,
            )
        })?;
        Ok(HipProgram { handle, raw: Arc::clone(&self.raw) })
    }

    fn epilogue_handle(&self, program: &ValidatedProgram) -> Result<Arc<HipProgram>, BackendError> {
        let key = program.content_hash();
        let mut cache = self.epilogues.lock().map_err(|_| BackendError::ExecutionFailed)?;
        if let Some(found) = cache.get(&key) {
            return Ok(Arc::clone(found));
        }
        let prepared = Arc::new(self.prepare_raw(program)?);
        cache.insert(key, Arc::clone(&prepared));
        Ok(prepared)
    }

    /// Lowers one validated dispatch (`Op`, crates/forja-core/src/ops.rs:163-302).  The Metal
    /// tuning attributes of argmax, top-k and sampling (`chunk_width`, `fast_top_k`, ...) are
    /// checked by forja-core when the dispatch is recorded and do not cross the boundary.
    fn lower_dispatch(
        &self,
        registry: &AllocationRegistry<HipBuffer>,
        dispatch: &Dispatch,
        keep: &mut Vec<Arc<HipProgram>>,
    ) -> Result<fh_dispatch, BackendError> {
        let mut lowered = fh_dispatch::default();
        match dispatch.op() {
            Op::Program(_) => {
                lowered.op = ffi::FH_OP_PROGRAM;
                let prepared = dispatch.prepared_program().ok_or(BackendError::ExecutionFailed)?;
                let handle =
                    prepared.backend_handle::<HipProgram>().ok_or(BackendError::InvalidInput)?;
                lowered.program = handle.handle;
            }
            Op::Copy => lowered.op = ffi::FH_OP_COPY,
            Op::PagedCopy { direction, start, page_tokens } => {
                lowered.op = ffi::FH_OP_PAGED_COPY;
                lowered.direction = match direction {
                    PagedCopyDirection::IntoPages => 0,
                    PagedCopyDirection::OutOfPages => 1,
                };
                lowered.start = start;
                lowered.page_tokens = page_tokens;
            }
            Op::RmsNorm { eps } => {
                lowered.op = ffi::FH_OP_RMS_NORM;
                lowered.eps = eps;
            }
            Op::Argmax { .. } => lowered.op = ffi::FH_OP_ARGMAX,
            Op::TopK { k, normalize, .. } => {
                lowered.op = ffi::FH_OP_TOP_K;
                lowered.k = k;
                lowered.normalize = u32::from(normalize);
            }
            Op::Sample { position, .. } => {
                lowered.op = ffi::FH_OP_SAMPLE;
                lowered.start = position;
            }
            Op::SampleMasked { position, .. } => {
                lowered.op = ffi::FH_OP_SAMPLE_MASKED;
                lowered.start = position;
            }
            Op::Rope { theta } => {
                lowered.op = ffi::FH_OP_ROPE;
                lowered.theta = theta;
            }
            Op::QuantEmbed { bits, group_size } => {
                lowered.op = ffi::FH_OP_QUANT_EMBED;
                lowered.bits = u32::from(bits);
                lowered.group_size = group_size;
            }
            Op::Matmul => lowered.op = ffi::FH_OP_MATMUL,
            Op::QuantMatmul { bits, group_size } => {
                lowered.op = ffi::FH_OP_QUANT_MATMUL;
                lowered.bits = u32::from(bits);
                lowered.group_size = group_size;
            }
            Op::GatherQuantMatmul { bits, group_size } => {
                lowered.op = ffi::FH_OP_GATHER_QUANT_MATMUL;
                lowered.bits = u32::from(bits);
                lowered.group_size = group_size;
            }
            Op::PagedSdpaAppend { scale, q_start, page_tokens } => {
                lowered.op = ffi::FH_OP_PAGED_SDPA_APPEND;
                lowered.scale = scale;
                lowered.q_start = q_start;
                lowered.page_tokens = page_tokens;
            }
            Op::PagedSdpa { scale, causal, q_start, key_length, page_tokens } => {
                lowered.op = ffi::FH_OP_PAGED_SDPA;
                lowered.scale = scale;
                lowered.causal = u32::from(causal);
                lowered.q_start = q_start;
                lowered.key_length = key_length;
                lowered.page_tokens = page_tokens;
            }
            // Outside the ragged forward step of the quantised engines: recurrent state, dense
            // embedding tables, dense routed products and contiguous-cache attention.
            Op::State(_) | Op::Embed | Op::GatherMatmul | Op::Sdpa { .. } => {
                return Err(BackendError::UnsupportedOperation);
            }
        }
        let inputs = dispatch.inputs();
        let outputs = dispatch.outputs();
        if inputs.len() > ffi::FH_MAX_INPUTS || outputs.len() > ffi::FH_MAX_OUTPUTS {
            return Err(BackendError::InvalidInput);
        }
        for (slot, tensor) in lowered.inputs.iter_mut().zip(inputs) {
            *slot = Self::lower_tensor(registry, tensor)?;
        }
        for (slot, tensor) in lowered.outputs.iter_mut().zip(outputs) {
            *slot = Self::lower_tensor(registry, tensor)?;
        }
        lowered.n_inputs = u32::try_from(inputs.len()).map_err(|_| BackendError::InvalidInput)?;
        lowered.n_outputs = u32::try_from(outputs.len()).map_err(|_| BackendError::InvalidInput)?;
        if let Some(epilogue) = dispatch.prepared_epilogue() {
            let handle = self.epilogue_handle(epilogue.validated())?;
            lowered.epilogue = handle.handle;
            lowered.accumulator_count = u32::from(epilogue.signature().accumulator_count());
            lowered.n_extras =
                u32::try_from(inputs.len() - dispatch.primitive_inputs().len())
                    .map_err(|_| BackendError::InvalidInput)?;
            keep.push(handle);
        }
        Ok(lowered)
    }

    fn submit_owned(
        &self,
        commands: CommandList,
        owners: Vec<CompletionResource>,
        profiled: bool,
    ) -> Result<HipSubmission, BackendError> {
        let dispatches = commands.into_dispatches();
        let mut keep = Vec::new();
        let lowered = {
            let registry = self.registry()?;
            dispatches
                .iter()
                .map(|dispatch| self.lower_dispatch(&registry, dispatch, &mut keep))
                .collect::<Result<Vec<_>, _>>()?
        };
        let count = u32::try_from(lowered.len()).map_err(|_| BackendError::InvalidInput)?;
        let mut raw = std::ptr::null_mut();
        check(unsafe {
            if profiled {
                ffi::fh_submit_profiled(self.raw.ptr(), lowered.as_ptr(), count, &mut raw)
            } else {
                ffi::fh_submit(self.raw.ptr(), lowered.as_ptr(), count, &mut raw)
            }
        })?;
        Ok(HipSubmission {
            raw: NonNull::new(raw).ok_or(BackendError::ExecutionFailed)?,
            _backend: Arc::clone(&self.raw),
            dispatches,
            profiled,
            _programs: keep,
            _owners: owners,
        })
    }
}

/// Completion handle of one submission.  It keeps the dispatches (and through them their
/// tensors' prepared programs), the epilogue handles and the caller's resources alive until the
/// device is done with them (crates/forja-core/src/backend.rs:14-26).
pub struct HipSubmission {
    raw: NonNull<ffi::fh_submission>,
    _backend: Arc<RawBackend>,
    dispatches: Vec<Dispatch>,
    profiled: bool,
    _programs: Vec<Arc<HipProgram>>,
    _owners: Vec<CompletionResource>,
}

unsafe impl Send for HipSubmission {}
unsafe impl Sync for HipSubmission {}

impl HipSubmission {
    fn wait_for(&self, timeout_ns: u64) -> Result<(), BackendError> {
        let mut error = fh_error::default();
        let status = unsafe { ffi::fh_wait(self.raw.as_ptr(), timeout_ns, &mut error) };
        if status == ffi::FH_OK { Ok(()) } else { Err(backend_error(status, &error)) }
    }
}

impl Submission for HipSubmission {
    fn wait(&self) -> Result<(), BackendError> {
        self.wait_for(0)
    }

    fn wait_timeout(&self, timeout: Duration) -> Result<(), BackendError> {
        // 0 means "no deadline" at the C ABI: an elapsed deadline still polls once.
        self.wait_for(u64::try_from(timeout.as_nanos()).unwrap_or(u64::MAX).max(1))
    }

    fn gpu_time(&self) -> Option<Duration> {
        match unsafe { ffi::fh_gpu_time_ns(self.raw.as_ptr()) } {
            0 => None,
            nanoseconds => Some(Duration::from_nanos(nanoseconds)),
        }
    }

    /// Per-dispatch device timeline of a submission made by `submit_profiled_retained`, after a
    /// successful wait (crates/forja-core/src/backend.rs:455-579).  The library times every
    /// dispatch it executes; dispatches it executed as one group (per-lane attention fused into
    /// one ragged launch) share the group's interval, the first member carrying `gap_before`.
    /// Costs are the logical ones of `KernelCost::of`; this backend has no variant catalog, no
    /// admission forecast and no padded-flop accounting, so those fields stay empty.
    fn profile(&self) -> Option<SubmissionProfile> {
        if !self.profiled {
            return None;
        }
        let mut count = 0_u32;
        let status = unsafe {
            ffi::fh_submission_profile(self.raw.as_ptr(), std::ptr::null_mut(), 0, &mut count)
        };
        if status != ffi::FH_OK {
            return None; // not waited for yet
        }
        let mut timings = vec![ffi::fh_dispatch_timing::default(); count as usize];
        let status = unsafe {
            ffi::fh_submission_profile(self.raw.as_ptr(), timings.as_mut_ptr(), count, &mut count)
        };
        if status != ffi::FH_OK {
            return None;
        }
        let mut per_dispatch = Vec::with_capacity(self.dispatches.len());
        let mut previous_end = Duration::ZERO;
        for timing in &timings {
            let start = Duration::from_nanos(timing.start_ns);
            let end = Duration::from_nanos(timing.end_ns);
            let first = timing.dispatch as usize;
            let members = self.dispatches.get(first..first + timing.dispatches as usize)?;
            for (nth, dispatch) in members.iter().enumerate() {
                let cost = KernelCost::of(dispatch).unwrap_or_default();
                per_dispatch.push(DispatchProfile {
                    scope: dispatch.profile_scope().map(|scope| (**scope).clone()),
                    op: dispatch.op(),
                    kernel: operation_name(timing.op),
                    variant: None,
                    alternatives: Vec::new(),
                    physical_dispatches: u64::from(nth == 0),
                    physical_threadgroups: 0,
                    predicted_gpu: Duration::ZERO,
                    compute_dtype: DType::F32,
                    cost,
                    scheduled_cost: cost,
                    critical_path_cost: KernelCost::default(),
                    padded_flops: [cost.flops, cost.flops],
                    inputs: dispatch.inputs().iter().map(ProfileTensor::from).collect(),
                    outputs: dispatch.outputs().iter().map(ProfileTensor::from).collect(),
                    barrier: true, // one in-order stream: every dispatch follows the one before
                    gpu_start: start,
                    gpu_end: end,
                    gap_before: if nth == 0 { start.saturating_sub(previous_end) } else { Duration::ZERO },
                    gpu_time: if nth == 0 { end.saturating_sub(start) } else { Duration::ZERO },
                    internal: Vec::new(),
                });
            }
            previous_end = end;
        }
        Some(SubmissionProfile {
            command_buffers: 1,
            gpu_time: self.gpu_time().unwrap_or_default(),
            dispatches: self.dispatches.len() as u64,
            barriers: self.dispatches.len().saturating_sub(1) as u64,
            per_dispatch,
            ..SubmissionProfile::default()
        })
    }
}

impl Drop for HipSubmission {
    fn drop(&mut self) {
        // Waits for the work when nobody did, so that the resources dropped after this are free.
        unsafe { ffi::fh_submission_free(self.raw.as_ptr()) }
    }
}

impl Backend for HipBackend {
    type Submission = HipSubmission;
    type ProgramHandle = HipProgram;

    fn memory_usage(&self) -> MemoryUsage {
        let mut bytes = 0;
        let status = unsafe { ffi::fh_memory_usage(self.raw.ptr(), &mut bytes) };
        if status != ffi::FH_OK {
            return MemoryUsage::default();
        }
        // every device byte the library holds for this backend, kept operands of the prefill
        // products and workspaces included
        MemoryUsage { charged_bytes: bytes, device_bytes: Some(bytes), ..MemoryUsage::default() }
    }

    fn set_memory_limit(&self, bytes: u64) {
        // the quota covers allocations and kept operands; the library evicts the latter first
        let _ = unsafe { ffi::fh_set_memory_limit(self.raw.ptr(), bytes) };
    }

    fn device_info(&self) -> Result<DeviceInfo, BackendError> {
        let mut info = std::mem::MaybeUninit::<ffi::fh_device_info>::zeroed();
        check(unsafe { ffi::fh_device_info_get(self.raw.ptr(), info.as_mut_ptr()) })?;
        let info = unsafe { info.assume_init() };
        let family: Vec<u8> =
            info.family.iter().take_while(|&&byte| byte != 0).map(|&byte| byte as u8).collect();
        Ok(DeviceInfo {
            family: String::from_utf8_lossy(&family).into_owned(),
            recommended_max_working_set_size: info.total_memory,
            max_threadgroup_memory_length: info.lds_bytes,
            gpu_core_count: Some(info.compute_units),
            simd_width: info.wavefront,
            // Published HBM3E rate of the part; `forja calibrate` replaces it with a measurement.
            streaming_read_gigabytes_per_second: 8000.0,
            streaming_copy_gigabytes_per_second: 8000.0,
        })
    }

    fn prepare_program(
        &self,
        program: &ValidatedProgram,
        _signature: &KernelSignature,
    ) -> Result<Self::ProgramHandle, BackendError> {
        self.prepare_raw(program)
    }

    fn alloc(&self, dtype: DType, shape: &[u32]) -> Result<Tensor, BackendError> {
        let elements = shape
            .iter()
            .try_fold(1_u64, |count, &extent| count.checked_mul(u64::from(extent)))
            .ok_or(BackendError::AllocationFailed)?;
        let byte_len =
            elements.checked_mul(dtype.byte_size()).ok_or(BackendError::AllocationFailed)?;
        let layout = Layout::contiguous(dtype, 0, shape.to_vec(), byte_len)
            .map_err(|_| BackendError::InvalidInput)?;
        let mut handle = 0;
        check(unsafe { ffi::fh_alloc(self.raw.ptr(), byte_len, &mut handle) })?;
        let mut registry = self.registry()?;
        let buffer =
            registry.insert(HipBuffer { handle, raw: Arc::clone(&self.raw) }, byte_len)?;
        registry.tensor(buffer, layout)
    }

    fn import_readonly(&self, bytes: MappedRegion) -> Result<ReadonlyImport, BackendError> {
        let byte_len = u64::try_from(bytes.len()).map_err(|_| BackendError::AllocationFailed)?;
        let mut handle = 0;
        check(unsafe {
            ffi::fh_import(self.raw.ptr(), bytes.as_ptr().cast(), byte_len, &mut handle)
        })?;
        // The bytes now live in HBM; the mapping is not kept.
        let buffer = self
            .registry()?
            .insert_read_only(HipBuffer { handle, raw: Arc::clone(&self.raw) }, byte_len)?;
        Ok(ReadonlyImport::Copied(buffer))
    }

    fn read_buffer_range(
        &self,
        buffer: BufferId,
        range: Range<u64>,
    ) -> Result<Vec<u8>, BackendError> {
        if range.end < range.start {
            return Err(BackendError::InvalidInput);
        }
        let handle = self.registry()?.get_buffer(buffer)?.handle;
        let len = usize::try_from(range.end - range.start).map_err(|_| BackendError::InvalidInput)?;
        let mut bytes = vec![0_u8; len];
        check(unsafe {
            ffi::fh_read(
                self.raw.ptr(),
                handle,
                range.start,
                bytes.as_mut_ptr().cast(),
                range.end - range.start,
            )
        })?;
        Ok(bytes)
    }

    fn tensor(&self, buffer: BufferId, layout: Layout) -> Result<Tensor, BackendError> {
        self.registry()?.tensor(buffer, layout)
    }

    fn view(&self, tensor: &Tensor, op: ViewOp) -> Result<Tensor, BackendError> {
        let layout = match op {
            ViewOp::Slice(spec) => tensor.layout().slice(&spec),
            ViewOp::Reshape(shape) => tensor.layout().reshape(&shape),
            ViewOp::Permute(axes) => tensor.layout().permute(&axes),
            ViewOp::Broadcast(shape) => tensor.layout().broadcast(&shape),
        }
        .map_err(|_| BackendError::InvalidInput)?;
        self.registry()?.view(tensor, layout)
    }

    fn write(&self, tensor: &Tensor, bytes: &[u8]) -> Result<(), BackendError> {
        let layout = tensor.layout();
        let expected = layout
            .element_count()
            .checked_mul(layout.dtype().byte_size())
            .ok_or(BackendError::InvalidInput)?;
        if !tensor.is_writable()
            || !layout.is_contiguous()
            || u64::try_from(bytes.len()).map_err(|_| BackendError::InvalidInput)? != expected
        {
            return Err(BackendError::InvalidInput);
        }
        let handle = self.registry()?.get(tensor)?.handle;
        check(unsafe {
            ffi::fh_write(
                self.raw.ptr(),
                handle,
                layout.byte_span().start,
                bytes.as_ptr().cast(),
                expected,
            )
        })
    }

    fn read(&self, tensor: &Tensor) -> Result<Vec<u8>, BackendError> {
        let lowered = Self::lower_tensor(&*self.registry()?, tensor)?;
        let layout = tensor.layout();
        let byte_len = layout
            .element_count()
            .checked_mul(layout.dtype().byte_size())
            .ok_or(BackendError::InvalidInput)?;
        let mut bytes =
            vec![0_u8; usize::try_from(byte_len).map_err(|_| BackendError::InvalidInput)?];
        check(unsafe {
            ffi::fh_read_tensor(self.raw.ptr(), &lowered, bytes.as_mut_ptr().cast(), byte_len)
        })?;
        Ok(bytes)
    }

    fn release(&self, tensor: &Tensor) -> Result<(), BackendError> {
        // Dropping the storage releases the device allocation (fh_release waits for the stream).
        drop(self.registry()?.remove(tensor)?);
        Ok(())
    }

    fn submit(&self, commands: CommandList) -> Result<Self::Submission, BackendError> {
        self.submit_owned(commands, Vec::new(), false)
    }

    fn submit_retained(
        &self,
        commands: CommandList,
        owners: Vec<CompletionResource>,
    ) -> Result<Self::Submission, BackendError> {
        self.submit_owned(commands, owners, false)
    }

    fn submit_profiled_retained(
        &self,
        commands: CommandList,
        owners: Vec<CompletionResource>,
    ) -> Result<Self::Submission, BackendError> {
        // one device timer per executed dispatch; read back by `Submission::profile`
        self.submit_owned(commands, owners, true)
    }
}

#[cfg(test)]
mod tests {
    use super::*;
    use forja_core::Slice;

    /// crates/forja-cpu/src/lib.rs:2786-2845 on the device: words 0, 0x11111111 and
    /// 0x11111111 * 15 dequantise to bias, scale + bias and 15 scale + bias.
    #[test]
    fn quant_matmul_dequantizes_q4_in_mlx_order() {
        let Ok(backend) = HipBackend::new(0) else { return };
        let rows = 7_u32;
        let x = backend.alloc(DType::BF16, &[rows, 64]).unwrap();
        let ones: Vec<u8> = std::iter::repeat([0x80_u8, 0x3f]).take(7 * 64).flatten().collect();
        backend.write(&x, &ones).unwrap();
        let packed = backend.alloc(DType::U32, &[3, 8]).unwrap();
        let words: Vec<u8> = [0_u32, 0x1111_1111, 0x1111_1111 * 15]
            .iter()
            .flat_map(|word| std::iter::repeat(word.to_le_bytes()).take(8).flatten())
            .collect();
        backend.write(&packed, &words).unwrap();
        let scales = backend.alloc(DType::BF16, &[3, 1]).unwrap();
        let biases = backend.alloc(DType::BF16, &[3, 1]).unwrap();
        backend.write(&scales, &[0x00, 0x3f, 0x00, 0x3f, 0x00, 0x3f]).unwrap(); // 0.5
        backend.write(&biases, &[0x80, 0x3e, 0x80, 0x3e, 0x80, 0x3e]).unwrap(); // 0.25
        let out = backend.alloc(DType::BF16, &[rows, 3]).unwrap();
        let mut commands = CommandList::new();
        commands
            .dispatch(Op::QuantMatmul { bits: 4, group_size: 64 }, &[&x, &packed, &scales, &biases], &out)
            .unwrap();
        backend.submit(commands).unwrap().wait().unwrap();
        let bytes = backend.read(&out).unwrap();
        let values: Vec<f32> = bytes
            .chunks_exact(2)
            .map(|pair| f32::from_bits(u32::from(u16::from_le_bytes([pair[0], pair[1]])) << 16))
            .collect();
        for row in values.chunks_exact(3) {
            assert_eq!(row, [16.0, 48.0, 496.0]); // 64 * (0.25, 0.75, 7.75)
        }
        let column = backend
            .view(&out, ViewOp::Slice(vec![Slice::new(0, rows, 1).unwrap(), Slice::new(1, 1, 1).unwrap()]))
            .unwrap();
        assert_eq!(backend.read(&column).unwrap().len(), 14);
        backend.release(&out).unwrap();
        assert_eq!(backend.read(&out), Err(BackendError::InvalidInput));
    }
}
