//! HipBackend — implements [`Backend`] on libfastnn_hip (hand-written HIP kernels for MI355X / gfx950).
//! Goes to `src/backend/hip/mod.rs` of the fastnn tree, behind the cargo feature `hip`
//! (`#[cfg(feature = "hip")] pub mod hip;` in src/backend/mod.rs next to the `wgpu` module, line 139-141).
//!
//! # Design
//!
//! - **compile()** reuses [`CpuBackend::compile`], as `WgpuBackend` does (src/backend/wgpu/mod.rs:119-130): the
//!   lowering is backend-agnostic, so kernel names (`matmul_i4`, `conv2d_i8_silu`, `quantize_activations`, ...),
//!   params and weight metas are exactly what `CpuBackend::dispatch` expects.
//! - **Buffer** is a token: the arena lives in device memory inside the native backend object
//!   (`fnn_backend_allocate_arena`), so activations never cross PCIe between instructions.  `write_arena` /
//!   `read_arena` are the only host <-> device copies of a pass (graph inputs and outputs).
//! - **dispatch()** mirrors the `ExecutablePlan` once into a native plan (`fnn_plan_add_*`), cached by a fingerprint
//!   of the instruction stream, and runs it with the call's `ShapeEnv`.  While a plan's constants stay in place the
//!   library skips every `WriteConst` and replays the whole instruction stream as one HIP graph.
//! - A kernel without a GPU implementation ends a dispatch segment with `UnsupportedOp` and the instruction's index;
//!   that one instruction runs on `CpuBackend` over a copy of the byte range it touches, exactly the way
//!   `WgpuBackend` falls back (src/backend/wgpu/mod.rs:162-239), and the dispatch resumes behind it.
//!
//! # GPU kernels
//!
//! `matmul_{i8,i4,u8,u4,f8,f8r,f4}[_relu|_gelu|_silu]` (codebook weights included), `matmul_i8_i8`, `matmul_i4_i8`,
//! `quantize_activations`, `dequantize_activations` (per tensor), `conv2d_{i8,i4,u8,u4,f8,f8r,f4}[_act]`,
//! `conv2d_{i8,i4}_i8[_act]`, `add_f32`, `relu_f32`, `gelu_f32`, `silu_f32`, `concat`, `slice_f32`, `pool_f32`,
//! `upsample_nearest2d`, plus `Fill`, `MemCopy`, `WriteConst`.  Everything else: CPU fallback per instruction.

mod ffi;

use crate::backend::cpu::{CpuBackend, CpuBuffer};
use crate::backend::{
    Backend, BackendError, BufferSlice, ExecutablePlan, Instruction, MemoryPlan, ProfileEntry,
};
use crate::ir::node::{ComputeGraph, DimExpr, ShapeEnv};
use std::cell::RefCell;
use std::collections::hash_map::DefaultHasher;
use std::ffi::{CStr, CString};
use std::hash::{Hash, Hasher};
use std::os::raw::{c_char, c_int, c_void};
use std::sync::Arc;

/// The arena of a [`HipBackend`]: device memory owned by the native backend object.  The value only records the
/// size the executor asked for (`GraphExecutor` re-allocates when a plan needs more, src/backend/executor.rs:66-72).
pub struct HipBuffer {
    bytes: usize,
}

impl HipBuffer {
    pub fn len(&self) -> usize {
        self.bytes
    }
    pub fn is_empty(&self) -> bool {
        self.bytes == 0
    }
}

/// One mirrored plan: the native handle and the symbol names its `param_dims` mention (the only entries of a
/// `ShapeEnv` the library needs to see).
struct Lowered {
    fingerprint: u64,
    raw: *mut ffi::fnn_plan,
    symbols: Vec<CString>,
}

impl Drop for Lowered {
    fn drop(&mut self) {
        // SAFETY: `raw` came from fnn_plan_create and is destroyed exactly once; every dispatch ends with a
        // stream synchronisation, so nothing on the device still refers to the plan.
        unsafe { ffi::fnn_plan_destroy(self.raw) }
    }
}

/// GPU backend on one MI355X.  One backend = one device context, one HIP stream, one device arena; like
/// `CpuBackend::dispatch` it is driven by one thread at a time.
pub struct HipBackend {
    raw: *mut ffi::fnn_backend,
    /// mirrored plans, most recently used last; the executor rewrites slice sizes of a plan with symbolic shapes
    /// between runs (src/backend/executor.rs:1218-1240), each distinct instruction stream is mirrored once
    plans: RefCell<Vec<Lowered>>,
}

/// How many mirrored plans are kept (a model has one plan per distinct set of runtime shapes).
const PLAN_CACHE: usize = 8;

// SAFETY: the native backend holds no thread-local state; it must only be *used* by one thread at a time, which
// `&mut GraphExecutor` / the Python GIL already guarantee for `CpuBackend` users.  On a multi-GPU host the calling
// thread's current HIP device must be the backend's device (the library sets it when it allocates).
unsafe impl Send for HipBackend {}

impl HipBackend {
    /// Opens device `device` (0 on a one-GPU box).  `Err(BackendError::Memory)` when no HIP device is present.
    pub fn new(device: i32) -> Result<Self, BackendError> {
        let mut raw: *mut ffi::fnn_backend = std::ptr::null_mut();
        // SAFETY: `raw` is a valid out-pointer; on failure the library leaves it null.
        let st = unsafe { ffi::fnn_backend_create(device as c_int, &mut raw) };
        if st != ffi::FNN_OK {
            return Err(error_from(st, std::ptr::null()));
        }
        Ok(HipBackend {
            raw,
            plans: RefCell::new(Vec::new()),
        })
    }

    /// Number of HIP devices the library sees (0 without a GPU or driver).
    pub fn device_count() -> usize {
        // SAFETY: no arguments, no state.
        unsafe { ffi::fnn_hip_device_count().max(0) as usize }
    }

    /// Rounds activations to f16 once on the matrix-core paths (agreement 1e-3 instead of 2e-5, about a third
    /// less time at M >= 64).  Off by default.
    pub fn set_fast_activations(&self, on: bool) -> Result<(), BackendError> {
        let flags = if on { ffi::FNN_FLAG_ACT_F16_SINGLE } else { 0 };
        // SAFETY: `self.raw` is live for the lifetime of `self`.
        self.check(unsafe { ffi::fnn_backend_set_kernel_flags(self.raw, flags) })
    }

    fn check(&self, st: c_int) -> Result<(), BackendError> {
        if st == ffi::FNN_OK {
            Ok(())
        } else {
            Err(error_from(st, self.raw))
        }
    }

    /// The native mirror of `plan`, built on first sight.
    fn lowered(&self, plan: &ExecutablePlan) -> Result<(*mut ffi::fnn_plan, Vec<*const c_char>, Vec<String>), BackendError> {
        let fp = fingerprint(plan);
        let mut plans = self.plans.borrow_mut();
        let pos = match plans.iter().position(|l| l.fingerprint == fp) {
            Some(i) => i,
            None => {
                if plans.len() >= PLAN_CACHE {
                    plans.remove(0);
                }
                plans.push(lower(plan, fp)?);
                plans.len() - 1
            }
        };
        // most recently used last
        let l = plans.remove(pos);
        plans.push(l);
        let l = plans.last().expect("just pushed");
        let ptrs = l.symbols.iter().map(|s| s.as_ptr()).collect();
        let names = l
            .symbols
            .iter()
            .map(|s| s.to_string_lossy().into_owned())
            .collect();
        Ok((l.raw, ptrs, names))
    }

    /// Runs instruction `index` of `plan` on `CpuBackend` over a copy of the byte range it touches and writes its
    /// outputs back to the device arena (the fallback of src/backend/wgpu/mod.rs:162-239).
    fn run_on_cpu(&self, plan: &ExecutablePlan, index: usize, shape_env: &ShapeEnv) -> Result<(), BackendError> {
        let Instruction::CallKernel {
            kernel_name,
            input_slices,
            output_slice,
            secondary_output_slice,
            params,
            node_id,
            param_dims,
            weight_meta,
        } = &plan.instructions[index]
        else {
            return Err(BackendError::Dispatch(format!(
                "hip: instruction {index} is not a CallKernel, yet the library refused it"
            )));
        };
        let arena_len = plan.arena_size;
        let clamp_end = |s: &BufferSlice| (s.offset + s.size).min(arena_len);
        let mut min_offset = output_slice.offset;
        let mut max_end = clamp_end(output_slice);
        for s in input_slices.iter().chain(secondary_output_slice.iter()) {
            min_offset = min_offset.min(s.offset);
            max_end = max_end.max(clamp_end(s));
        }
        let range_len = max_end - min_offset;
        let mut tmp = vec![0u8; range_len];
        // SAFETY: `tmp` holds `range_len` writable bytes; the range lies inside the arena (checked by the library).
        self.check(unsafe {
            ffi::fnn_backend_read_arena(self.raw, min_offset as u64, tmp.as_mut_ptr() as *mut c_void, range_len as u64)
        })?;
        let shift = |s: &BufferSlice| BufferSlice {
            offset: s.offset - min_offset,
            size: s.size,
        };
        let single = ExecutablePlan {
            instructions: vec![Instruction::CallKernel {
                kernel_name: kernel_name.clone(),
                input_slices: input_slices.iter().map(shift).collect(),
                output_slice: shift(output_slice),
                secondary_output_slice: secondary_output_slice.as_ref().map(shift),
                params: params.clone(),
                node_id: *node_id,
                param_dims: param_dims.clone(),
                weight_meta: weight_meta.clone(),
            }],
            arena_size: range_len,
            levels: vec![0],
        };
        let cpu_buf = CpuBuffer::new(tmp);
        CpuBackend.dispatch(&single, &cpu_buf, shape_env)?;
        let data = cpu_buf.data_mut();
        for s in std::iter::once(output_slice).chain(secondary_output_slice.iter()) {
            let (a, e) = (s.offset - min_offset, clamp_end(s) - min_offset);
            // SAFETY: `data[a..e]` is a live slice of `e - a` bytes; the destination range lies inside the arena.
            self.check(unsafe {
                ffi::fnn_backend_write_arena(self.raw, s.offset as u64, data[a..e].as_ptr() as *const c_void, (e - a) as u64)
            })?;
        }
        Ok(())
    }
}

impl Drop for HipBackend {
    fn drop(&mut self) {
        self.plans.borrow_mut().clear(); // plans first: their graphs belong to this backend's context
        // SAFETY: `raw` came from fnn_backend_create and is destroyed exactly once.
        unsafe { ffi::fnn_backend_destroy(self.raw) }
    }
}

/// Kernel names of the weight-quantised MatMul with f32 activations (src/backend/cpu/mod.rs:459-495).  The
/// I8-activation forms (`matmul_i8_i8`, `matmul_i4_i8`) have no fused epilogue on either backend.
const QUANTISED_MATMULS: [&str; 7] =
    ["matmul_i8", "matmul_i4", "matmul_u8", "matmul_u4", "matmul_f8", "matmul_f8r", "matmul_f4"];

/// Suffix for a node's `fused_op`, with the mapping of `activation_type` in src/backend/cpu/mod.rs:408-413.
fn epilogue_suffix(fused_op: Option<&str>) -> &'static str {
    match fused_op {
        Some("MatMulAddRelu") | Some("OpRelu") => "_relu",
        Some("MatMulAddGelu") | Some("OpGelu") => "_gelu",
        Some("MatMulAddSilu") | Some("OpSilu") => "_silu",
        _ => "",
    }
}

/// Appends `_relu` / `_gelu` / `_silu` to every quantised MatMul whose graph node carries a fused activation.
/// Instructions without a `node_id`, nodes that are gone and every other kernel are left as they are.
fn tag_matmul_epilogues(plan: &mut ExecutablePlan, graph: &ComputeGraph) {
    for ins in plan.instructions.iter_mut() {
        if let Instruction::CallKernel { kernel_name, node_id: Some(id), .. } = ins {
            if !QUANTISED_MATMULS.contains(&kernel_name.as_str()) {
                continue;
            }
            let fused = graph.get_node(*id).and_then(|n| n.attrs.get("fused_op")).map(|s| s.as_str());
            kernel_name.push_str(epilogue_suffix(fused));
        }
    }
}

impl Backend for HipBackend {
    type Buffer = HipBuffer;

    fn name(&self) -> &str {
        "hip"
    }

    /// The device arena is (re)allocated and zero-filled, like `CpuBuffer::new(vec![0; n])`.  The trait has no error
    /// channel here, so running out of device memory panics with the library's message, as `Vec` would on the host.
    fn allocate_arena(&self, total_bytes: usize) -> HipBuffer {
        // SAFETY: `self.raw` is live.
        if let Err(e) = self.check(unsafe { ffi::fnn_backend_allocate_arena(self.raw, total_bytes as u64) }) {
            panic!("hip: allocate_arena({total_bytes}): {e}");
        }
        HipBuffer { bytes: total_bytes }
    }

    /// `CpuBackend::compile`, then the fused epilogue of every quantised MatMul is carried in its kernel name.
    ///
    /// The CPU lowering works out `activation_type` from the node's `fused_op` attribute but names a quantised MatMul
    /// `matmul_i8` / `matmul_i4` / ... without it (src/backend/cpu/mod.rs:406-413, 427-495), so the instruction
    /// alone does not say that a ReLU / GELU / SiLU was folded into the node (`MatMulAdd{Relu,Gelu,Silu}`: the bias
    /// is the third input slice; `Op{Relu,Gelu,Silu}`: no bias).  Conv2d names already carry the tag
    /// (`conv2d_i8_silu`, src/backend/cpu/mod.rs:856-865); this gives MatMul the same form, which is what
    /// libfastnn_hip reads: `matmul_<type>[_relu|_gelu|_silu]`, bias = third slice when present.
    fn compile(&self, graph: &ComputeGraph, memory_plan: &MemoryPlan) -> Result<ExecutablePlan, BackendError> {
        let mut plan = CpuBackend.compile(graph, memory_plan)?;
        tag_matmul_epilogues(&mut plan, graph);
        Ok(plan)
    }

    fn dispatch(&self, plan: &ExecutablePlan, _arena: &HipBuffer, shape_env: &ShapeEnv) -> Result<(), BackendError> {
        let (native, symbol_ptrs, symbol_names) = self.lowered(plan)?;
        // the bindings of the symbols this plan mentions (an unbound Symbol is the library's error, with the
        // reference's text; an unbound Bounded dim falls back to its max there)
        let mut names: Vec<*const c_char> = Vec::new();
        let mut values: Vec<u64> = Vec::new();
        for (ptr, name) in symbol_ptrs.iter().zip(symbol_names.iter()) {
            if let Some(v) = shape_env.resolve(name) {
                names.push(*ptr);
                values.push(v);
            }
        }
        let mut first = 0u64;
        loop {
            let mut stopped = 0u64;
            // SAFETY: `native` is kept alive by `self.plans` (nothing evicts it before this call returns: the
            // cache is only touched by `lowered`); `names` / `values` hold `names.len()` entries each and the
            // CStrings behind `names` live in the same cache entry.
            let st = unsafe {
                ffi::fnn_backend_dispatch_from(
                    self.raw,
                    native,
                    names.as_ptr(),
                    values.as_ptr(),
                    names.len() as u64,
                    first,
                    &mut stopped,
                )
            };
            match st {
                ffi::FNN_OK => return Ok(()),
                ffi::FNN_ERR_UNSUPPORTED_OP => {
                    self.run_on_cpu(plan, stopped as usize, shape_env)?;
                    first = stopped + 1;
                }
                other => return Err(error_from(other, self.raw)),
            }
        }
    }

    /// Per-instruction timings from the library when every kernel of the plan runs on the GPU (each instruction is
    /// followed by a stream synchronisation); otherwise the trait's one-instruction-at-a-time default.
    fn dispatch_profile(
        &self,
        plan: &ExecutablePlan,
        arena: &HipBuffer,
        shape_env: &ShapeEnv,
    ) -> Result<Vec<ProfileEntry>, BackendError> {
        let (native, symbol_ptrs, symbol_names) = self.lowered(plan)?;
        let n = plan.instructions.len();
        let mut ns = vec![0u64; n.max(1)];
        // the same bindings `dispatch` passes: symbolic dims are profiled under this call's environment
        let mut names: Vec<*const c_char> = Vec::new();
        let mut values: Vec<u64> = Vec::new();
        for (ptr, name) in symbol_ptrs.iter().zip(symbol_names.iter()) {
            if let Some(v) = shape_env.resolve(name) {
                names.push(*ptr);
                values.push(v);
            }
        }
        // SAFETY: `ns` holds at least `n` entries; `names` / `values` hold `names.len()` entries each and the
        // CStrings behind `names` live in the plan cache entry that `native` belongs to.
        let st = unsafe {
            ffi::fnn_backend_dispatch_profile_env(
                self.raw,
                native,
                names.as_ptr(),
                values.as_ptr(),
                names.len() as u64,
                ns.as_mut_ptr(),
                n as u64,
            )
        };
        if st == ffi::FNN_ERR_UNSUPPORTED_OP {
            return default_profile(self, plan, arena, shape_env);
        }
        self.check(st)?;
        Ok(plan
            .instructions
            .iter()
            .enumerate()
            .map(|(i, ins)| {
                let (node_id, kernel_name) = match ins {
                    Instruction::CallKernel { node_id, kernel_name, .. } => (*node_id, kernel_name.clone()),
                    Instruction::MemCopy { .. } => (None, "memcopy".to_string()),
                    Instruction::Fill { .. } => (None, "fill".to_string()),
                    Instruction::WriteConst { .. } => (None, "write_const".to_string()),
                };
                ProfileEntry {
                    instruction_index: i,
                    node_id,
                    kernel_name,
                    elapsed_ns: ns[i] as u128,
                }
            })
            .collect())
    }

    fn write_arena(&self, arena: &HipBuffer, offset: usize, data: &[u8]) {
        // same clamping as CpuBackend / WgpuBackend (src/backend/wgpu/mod.rs:281-285)
        let end = (offset + data.len()).min(arena.bytes);
        if end <= offset {
            return;
        }
        // SAFETY: `data[..end - offset]` is a live slice.
        if let Err(e) = self.check(unsafe {
            ffi::fnn_backend_write_arena(self.raw, offset as u64, data.as_ptr() as *const c_void, (end - offset) as u64)
        }) {
            panic!("hip: write_arena: {e}");
        }
    }

    fn read_arena(&self, arena: &HipBuffer, offset: usize, size: usize) -> Vec<u8> {
        let end = (offset + size).min(arena.bytes);
        let mut out = vec![0u8; end.saturating_sub(offset)];
        if out.is_empty() {
            return out;
        }
        // SAFETY: `out` holds `out.len()` writable bytes.
        if let Err(e) = self.check(unsafe {
            ffi::fnn_backend_read_arena(self.raw, offset as u64, out.as_mut_ptr() as *mut c_void, out.len() as u64)
        }) {
            panic!("hip: read_arena: {e}");
        }
        out
    }
}

/// The trait's default `dispatch_profile` body (src/backend/mod.rs:178-211), for plans with CPU fallbacks.
fn default_profile(
    b: &HipBackend,
    plan: &ExecutablePlan,
    arena: &HipBuffer,
    shape_env: &ShapeEnv,
) -> Result<Vec<ProfileEntry>, BackendError> {
    let mut entries = Vec::with_capacity(plan.instructions.len());
    for (instruction_index, instruction) in plan.instructions.iter().cloned().enumerate() {
        let (node_id, kernel_name) = match &instruction {
            Instruction::CallKernel { node_id, kernel_name, .. } => (*node_id, kernel_name.clone()),
            Instruction::MemCopy { .. } => (None, "memcopy".to_string()),
            Instruction::Fill { .. } => (None, "fill".to_string()),
            Instruction::WriteConst { .. } => (None, "write_const".to_string()),
        };
        let single = ExecutablePlan {
            instructions: vec![instruction],
            arena_size: plan.arena_size,
            levels: vec![0],
        };
        let start = std::time::Instant::now();
        b.dispatch(&single, arena, shape_env)?;
        entries.push(ProfileEntry {
            instruction_index,
            node_id,
            kernel_name,
            elapsed_ns: start.elapsed().as_nanos(),
        });
    }
    Ok(entries)
}

/// Status code + the library's message -> `BackendError` (src/backend/mod.rs:6-12).
fn error_from(st: c_int, b: *const ffi::fnn_backend) -> BackendError {
    // SAFETY: fnn_backend_last_error accepts null and always returns a NUL-terminated string that stays valid until
    // the next call on the same backend / thread; it is copied at once.
    let msg = unsafe { CStr::from_ptr(ffi::fnn_backend_last_error(b)) }
        .to_string_lossy()
        .into_owned();
    match st {
        ffi::FNN_ERR_MEMORY => BackendError::Memory(msg),
        ffi::FNN_ERR_UNSUPPORTED_OP => BackendError::UnsupportedOp(msg),
        ffi::FNN_ERR_COMPILATION => BackendError::Compilation(msg),
        _ => BackendError::Dispatch(msg),
    }
}

/// Identity of an instruction stream: everything `lower` reads, with payloads by address and length (a `WriteConst`
/// payload or an `Arc<QuantizedWeightMeta>` is immutable once the plan exists).
fn fingerprint(plan: &ExecutablePlan) -> u64 {
    let mut h = DefaultHasher::new();
    plan.arena_size.hash(&mut h);
    plan.instructions.len().hash(&mut h);
    let slice = |s: &BufferSlice, h: &mut DefaultHasher| {
        s.offset.hash(h);
        s.size.hash(h);
    };
    for ins in &plan.instructions {
        match ins {
            Instruction::CallKernel {
                kernel_name,
                input_slices,
                output_slice,
                secondary_output_slice,
                params,
                param_dims,
                weight_meta,
                ..
            } => {
                0u8.hash(&mut h);
                kernel_name.hash(&mut h);
                for s in input_slices {
                    slice(s, &mut h);
                }
                slice(output_slice, &mut h);
                if let Some(s) = secondary_output_slice {
                    slice(s, &mut h);
                }
                params.hash(&mut h);
                if let Some(dims) = param_dims {
                    for d in dims {
                        match d {
                            DimExpr::Known(v) => (0u8, *v).hash(&mut h),
                            DimExpr::Symbol(s) => (1u8, s).hash(&mut h),
                            DimExpr::Bounded { sym, max } => (2u8, sym, *max).hash(&mut h),
                        }
                    }
                }
                if let Some(m) = weight_meta {
                    (Arc::as_ptr(m) as usize).hash(&mut h);
                }
            }
            Instruction::MemCopy { dst, src } => {
                1u8.hash(&mut h);
                slice(dst, &mut h);
                slice(src, &mut h);
            }
            Instruction::Fill { dst, value } => {
                2u8.hash(&mut h);
                slice(dst, &mut h);
                value.to_bits().hash(&mut h);
            }
            Instruction::WriteConst { dst, data } => {
                3u8.hash(&mut h);
                slice(dst, &mut h);
                (data.as_ptr() as usize, data.len()).hash(&mut h);
            }
        }
    }
    h.finish()
}

/// Mirrors every instruction of `plan` into a native plan (payloads are copied by the library).
fn lower(plan: &ExecutablePlan, fingerprint: u64) -> Result<Lowered, BackendError> {
    let mut raw: *mut ffi::fnn_plan = std::ptr::null_mut();
    // SAFETY: valid out-pointer.
    let st = unsafe { ffi::fnn_plan_create(plan.arena_size as u64, &mut raw) };
    if st != ffi::FNN_OK {
        return Err(error_from(st, std::ptr::null()));
    }
    let mut lowered = Lowered {
        fingerprint,
        raw,
        symbols: Vec::new(),
    }; // dropped (and the native plan destroyed) on every early return below
    let fs = |s: &BufferSlice| ffi::fnn_slice {
        offset: s.offset as u64,
        size: s.size as u64,
    };
    let ok = |st: c_int| -> Result<(), BackendError> {
        if st == ffi::FNN_OK {
            Ok(())
        } else {
            Err(error_from(st, std::ptr::null()))
        }
    };
    for (index, ins) in plan.instructions.iter().enumerate() {
        match ins {
            Instruction::WriteConst { dst, data } => {
                // SAFETY: `data` is a live slice of `data.len()` bytes; the library copies it.
                ok(unsafe { ffi::fnn_plan_add_write_const(raw, fs(dst), data.as_ptr() as *const c_void, data.len() as u64) })?;
            }
            Instruction::Fill { dst, value } => {
                // SAFETY: plain values.
                ok(unsafe { ffi::fnn_plan_add_fill(raw, fs(dst), *value) })?;
            }
            Instruction::MemCopy { dst, src } => {
                // SAFETY: plain values.
                ok(unsafe { ffi::fnn_plan_add_memcopy(raw, fs(dst), fs(src)) })?;
            }
            Instruction::CallKernel {
                kernel_name,
                input_slices,
                output_slice,
                secondary_output_slice,
                params,
                param_dims,
                weight_meta,
                node_id: _,
            } => {
                let name = CString::new(kernel_name.as_str())
                    .map_err(|_| BackendError::Dispatch(format!("hip: kernel name {kernel_name:?} contains a NUL byte")))?;
                let inputs: Vec<ffi::fnn_slice> = input_slices.iter().map(fs).collect();
                let secondary = secondary_output_slice.as_ref().map(fs);
                let params64: Vec<u64> = params.iter().map(|&p| p as u64).collect();
                // QuantizedWeightMeta flattened; the vectors outlive the call below, the library copies them
                let shape64: Vec<u64>;
                let codebooks: Vec<f32>;
                let meta = match weight_meta {
                    Some(m) => {
                        shape64 = m.shape.iter().map(|&d| d as u64).collect();
                        codebooks = m.codebooks.iter().flat_map(|cb| cb.iter().copied()).collect();
                        Some(ffi::fnn_weight_meta {
                            bit_width: m.bit_width as u64,
                            scales: m.scales.as_ptr(),
                            n_scales: m.scales.len() as u64,
                            zero_points: m.zero_points.as_ptr(),
                            n_zero_points: m.zero_points.len() as u64,
                            shape: shape64.as_ptr(),
                            n_shape: shape64.len() as u64,
                            quant_block_size: m.quant_block_size as u64,
                            codebooks: if codebooks.is_empty() { std::ptr::null() } else { codebooks.as_ptr() },
                            n_codebooks: m.codebooks.len() as u64,
                        })
                    }
                    None => None,
                };
                // SAFETY: every pointer refers to a live local (`name`, `inputs`, `params64`, `meta` and the
                // vectors it points into) holding the stated number of elements; null stands for None.
                ok(unsafe {
                    ffi::fnn_plan_add_call_kernel(
                        raw,
                        name.as_ptr(),
                        inputs.as_ptr(),
                        inputs.len() as u64,
                        fs(output_slice),
                        secondary.as_ref().map_or(std::ptr::null(), |s| s as *const ffi::fnn_slice),
                        params64.as_ptr(),
                        params64.len() as u64,
                        meta.as_ref().map_or(std::ptr::null(), |m| m as *const ffi::fnn_weight_meta),
                    )
                })?;
                if let Some(dims) = param_dims {
                    // symbol names live as CStrings for the duration of the call (the library copies them) and, once,
                    // in `lowered.symbols` for building the per-dispatch environment
                    let mut keep: Vec<CString> = Vec::new();
                    let mut native_dims: Vec<ffi::fnn_dim_expr> = Vec::with_capacity(dims.len());
                    for d in dims {
                        let (kind, value, sym) = match d {
                            DimExpr::Known(v) => (0u32, *v, None),
                            DimExpr::Symbol(s) => (1u32, 0u64, Some(s)),
                            DimExpr::Bounded { sym, max } => (2u32, *max, Some(sym)),
                        };
                        let ptr = match sym {
                            Some(s) => {
                                let c = CString::new(s.as_str())
                                    .map_err(|_| BackendError::Dispatch(format!("hip: symbol {s:?} contains a NUL byte")))?;
                                if !lowered.symbols.contains(&c) {
                                    lowered.symbols.push(c.clone());
                                }
                                keep.push(c);
                                keep.last().expect("just pushed").as_ptr()
                            }
                            None => std::ptr::null(),
                        };
                        native_dims.push(ffi::fnn_dim_expr { kind, value, symbol: ptr });
                    }
                    // SAFETY: `native_dims` holds `native_dims.len()` entries whose symbol pointers refer to the
                    // heap buffers of the CStrings in `keep` (moving a CString does not move its buffer).
                    ok(unsafe { ffi::fnn_plan_set_param_dims(raw, index as u64, native_dims.as_ptr(), native_dims.len() as u64) })?;
                }
            }
        }
    }
    Ok(lowered)
}
