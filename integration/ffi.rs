//! Raw bindings of libfastnn_hip's host-side backend (include/fastnn_hip_backend.h, include/fastnn_hip.h).
//! Goes to `src/backend/hip/ffi.rs` of the fastnn tree, behind the cargo feature `hip`.
//!
//! Every function returns an `fnn_status` (0 Ok, 1 Dispatch, 2 Memory, 3 UnsupportedOp, 4 Compilation: the variants
//! of `BackendError`, src/backend/mod.rs:6-12); the text of the last failure comes from `fnn_backend_last_error`.
//! Nothing unwinds across this boundary: the library catches C++ exceptions in every entry point.
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_int, c_void};

#[repr(C)]
pub struct fnn_backend {
    _private: [u8; 0],
}
#[repr(C)]
pub struct fnn_plan {
    _private: [u8; 0],
}

/// BufferSlice, src/backend/mod.rs:27-31
#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct fnn_slice {
    pub offset: u64,
    pub size: u64,
}

/// QuantizedWeightMeta, src/backend/mod.rs:40-58 (`codebooks`: `n_codebooks` x 16 floats, null when empty)
#[repr(C)]
pub struct fnn_weight_meta {
    pub bit_width: u64,
    pub scales: *const f32,
    pub n_scales: u64,
    pub zero_points: *const f32,
    pub n_zero_points: u64,
    pub shape: *const u64,
    pub n_shape: u64,
    pub quant_block_size: u64,
    pub codebooks: *const f32,
    pub n_codebooks: u64,
}

/// DimExpr, src/ir/node.rs:163-167: kind 0 Known(value), 1 Symbol(symbol), 2 Bounded { sym: symbol, max: value }
#[repr(C)]
pub struct fnn_dim_expr {
    pub kind: u32,
    pub value: u64,
    pub symbol: *const c_char,
}

pub const FNN_OK: c_int = 0;
pub const FNN_ERR_DISPATCH: c_int = 1;
pub const FNN_ERR_MEMORY: c_int = 2;
pub const FNN_ERR_UNSUPPORTED_OP: c_int = 3;
pub const FNN_ERR_COMPILATION: c_int = 4;

/// FNN_FLAG_ACT_F16_SINGLE of include/fastnn_hip.h (per-backend kernel flag: 1e-3 instead of 2e-5 agreement)
pub const FNN_FLAG_ACT_F16_SINGLE: c_int = 1 << 2;

extern "C" {
    pub fn fnn_hip_device_count() -> c_int;
    pub fn fnn_hip_version() -> *const c_char;

    pub fn fnn_backend_create(device: c_int, out: *mut *mut fnn_backend) -> c_int;
    pub fn fnn_backend_destroy(b: *mut fnn_backend);
    pub fn fnn_backend_name(b: *const fnn_backend) -> *const c_char;
    /// b may be null: the message of a failed `fnn_backend_create` / `fnn_plan_*` call on this thread
    pub fn fnn_backend_last_error(b: *const fnn_backend) -> *const c_char;
    pub fn fnn_backend_set_kernel_flags(b: *mut fnn_backend, flags: c_int) -> c_int;
    pub fn fnn_backend_set_graph_replay(b: *mut fnn_backend, enabled: c_int) -> c_int;
    pub fn fnn_backend_allocate_arena(b: *mut fnn_backend, total_bytes: u64) -> c_int;
    pub fn fnn_backend_write_arena(b: *mut fnn_backend, offset: u64, data: *const c_void, size: u64) -> c_int;
    pub fn fnn_backend_read_arena(b: *mut fnn_backend, offset: u64, out: *mut c_void, size: u64) -> c_int;

    pub fn fnn_plan_create(arena_size: u64, out: *mut *mut fnn_plan) -> c_int;
    pub fn fnn_plan_destroy(p: *mut fnn_plan);
    pub fn fnn_plan_len(p: *const fnn_plan) -> u64;
    pub fn fnn_plan_add_write_const(p: *mut fnn_plan, dst: fnn_slice, data: *const c_void, len: u64) -> c_int;
    pub fn fnn_plan_add_fill(p: *mut fnn_plan, dst: fnn_slice, value: f32) -> c_int;
    pub fn fnn_plan_add_memcopy(p: *mut fnn_plan, dst: fnn_slice, src: fnn_slice) -> c_int;
    pub fn fnn_plan_add_call_kernel(
        p: *mut fnn_plan,
        kernel_name: *const c_char,
        inputs: *const fnn_slice,
        n_inputs: u64,
        output: fnn_slice,
        secondary_output: *const fnn_slice, // null for None
        params: *const u64,
        n_params: u64,
        meta: *const fnn_weight_meta, // null for None
    ) -> c_int;
    pub fn fnn_plan_set_param_dims(p: *mut fnn_plan, instruction: u64, dims: *const fnn_dim_expr, n_dims: u64) -> c_int;
    pub fn fnn_plan_from_bincode(bytes: *const c_void, len: u64, out: *mut *mut fnn_plan) -> c_int;

    pub fn fnn_backend_dispatch_env(
        b: *mut fnn_backend,
        p: *mut fnn_plan,
        names: *const *const c_char,
        values: *const u64,
        n_symbols: u64,
    ) -> c_int;
    /// One segment of a dispatch: stops with status 3 and the index in `stopped_at` at a kernel the library does
    /// not implement; resume with `first = *stopped_at + 1`.
    pub fn fnn_backend_dispatch_from(
        b: *mut fnn_backend,
        p: *mut fnn_plan,
        names: *const *const c_char,
        values: *const u64,
        n_symbols: u64,
        first: u64,
        stopped_at: *mut u64,
    ) -> c_int;
    pub fn fnn_backend_dispatch_profile(b: *mut fnn_backend, p: *mut fnn_plan, elapsed_ns: *mut u64, n: u64) -> c_int;
    /// `fnn_backend_dispatch_profile` under the bindings of a `ShapeEnv`.
    pub fn fnn_backend_dispatch_profile_env(
        b: *mut fnn_backend,
        p: *mut fnn_plan,
        names: *const *const c_char,
        values: *const u64,
        n_symbols: u64,
        elapsed_ns: *mut u64,
        n: u64,
    ) -> c_int;
}
