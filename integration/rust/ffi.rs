//! `nabla-train/src/optim/mi355x/ffi.rs` -- the C ABI of `libnabla_optim.so` (`include/nabla_optim.h`).
//!
//! UNVERIFIED SOURCE: written against the header by hand; the image this was written in has no
//! Rust toolchain.  `tests/test_rust_shim.py` checks every declaration below against the header
//! (symbol names, number of arguments, integer / floating-point / pointer kind of each argument).
//!
//! Link with `println!("cargo:rustc-link-lib=dylib=nabla_optim");` in `nabla-train/build.rs`.
#![allow(non_camel_case_types, dead_code)]

use std::os::raw::{c_char, c_int, c_void};

#[repr(C)] pub struct NboMeta { pub kind: i32, pub reserved: i32, pub lr: f64, pub beta1: f64,
    pub beta2: f64, pub eps: f64, pub weight_decay: f64, pub momentum: f64, pub step_count: u64 }
#[repr(C)] pub struct NboScalerState { pub scale: f64, pub growth_factor: f64, pub backoff_factor: f64,
    pub growth_interval: u64, pub consecutive_ok: u64 }
#[repr(C)] pub struct NboStepInfo { pub scale: f64, pub norm: f64, pub step_count: u64,
    pub found_inf: u32, pub clipped: u32 }
pub enum NboList {} pub enum NboOptim {} pub enum NboScaler {} pub enum NboPlaced {}

pub const NBO_DT_F32: c_int = 0; pub const NBO_DT_BF16: c_int = 1; pub const NBO_DT_F64: c_int = 2;
pub const NBO_DT_F16: c_int = 3;
pub const NBO_KIND_ADAMW: i32 = 0; pub const NBO_KIND_ADAM: i32 = 1; pub const NBO_KIND_SGD: i32 = 2;
pub const NBO_STEP_ZERO_GRADS: u32 = 1; pub const NBO_STEP_SKIP_NONFINITE: u32 = 2;
pub const NBO_STEP_ZERO_ON_SKIP: u32 = 4;
pub const NBO_ACC_CHECK_FINITE: u32 = 1; pub const NBO_ACC_WRITE_GRADS: u32 = 2;
// nbo_status
pub const NBO_OK: c_int = 0; pub const NBO_ERR_LEN_MISMATCH: c_int = 1; pub const NBO_ERR_COUNT_MISMATCH: c_int = 2;
pub const NBO_ERR_SHAPE: c_int = 3; pub const NBO_ERR_STATE_KEY: c_int = 4; pub const NBO_ERR_STATE_INDEX: c_int = 5;
pub const NBO_ERR_KIND: c_int = 6;

#[link(name = "nabla_optim")]
extern "C" {
    pub fn nbo_init() -> c_int;
    pub fn nbo_set_stream(hip_stream: *mut c_void) -> c_int;
    pub fn nbo_sync() -> c_int;
    pub fn nbo_last_error() -> *const c_char;
    pub fn nbo_list_create(n: u64, rows: *const u64, cols: *const u64, dtype: c_int,
                           dev_ptrs: *const *const c_void, out: *mut *mut NboList) -> c_int;
    pub fn nbo_list_set_ptrs(list: *mut NboList, dev_ptrs: *const *const c_void) -> c_int;
    pub fn nbo_list_destroy(list: *mut NboList) -> c_int;
    pub fn nbo_optim_create(meta: *const NboMeta, n: u64, rows: *const u64, cols: *const u64,
                            state_dtype: c_int, keep_master: c_int, out: *mut *mut NboOptim) -> c_int;
    pub fn nbo_optim_destroy(opt: *mut NboOptim) -> c_int;
    pub fn nbo_optim_step(opt: *mut NboOptim, params: *mut NboList, grads: *mut NboList) -> c_int;
    pub fn nbo_optim_reset(opt: *mut NboOptim) -> c_int;
    pub fn nbo_optim_set_lr(opt: *mut NboOptim, lr: f64) -> c_int;
    pub fn nbo_optim_get_meta(opt: *mut NboOptim, out: *mut NboMeta) -> c_int;
    pub fn nbo_optim_load_meta(opt: *mut NboOptim, meta: *const NboMeta) -> c_int;
    pub fn nbo_optim_state_read(opt: *mut NboOptim, name: *const c_char, buf: *mut c_void,
                                n_elems: u64, on_device: c_int) -> c_int;
    pub fn nbo_optim_state_write(opt: *mut NboOptim, name: *const c_char, buf: *const c_void,
                                 n_elems: u64, on_device: c_int) -> c_int;
    pub fn nbo_optim_master_from_params(opt: *mut NboOptim, params_half: *mut NboList) -> c_int;
    pub fn nbo_optim_params_from_master(opt: *mut NboOptim, params_half: *mut NboList) -> c_int;
    pub fn nbo_scaler_create(state: *const NboScalerState, out: *mut *mut NboScaler) -> c_int;
    pub fn nbo_scaler_destroy(s: *mut NboScaler) -> c_int;
    pub fn nbo_scaler_state_get(s: *mut NboScaler, out: *mut NboScalerState) -> c_int;
    pub fn nbo_scaler_load_state(s: *mut NboScaler, state: *const NboScalerState) -> c_int;
    pub fn nbo_scaler_unscale_and_update(s: *mut NboScaler, grads: *mut NboList, ok: *mut c_int) -> c_int;
    pub fn nbo_clip_grad_norm(grads: *mut NboList, max_norm: f64, norm: *mut f64) -> c_int;
    pub fn nbo_zero_grad(grads: *mut NboList) -> c_int;
    pub fn nbo_scale_grad(grads: *mut NboList, factor: f64) -> c_int;
    pub fn nbo_fused_step(opt: *mut NboOptim, scaler: *mut NboScaler, params: *mut NboList,
                          grads: *mut NboList, max_norm: f64, flags: u32) -> c_int;
    // no counterpart in the reference: nbo_fused_step for callers that cannot allocate device memory
    pub fn nbo_fused_step_noalloc(opt: *mut NboOptim, scaler: *mut NboScaler, params: *mut NboList,
                                  grads: *mut NboList, max_norm: f64, flags: u32) -> c_int;
    pub fn nbo_optim_last_step(opt: *mut NboOptim, out: *mut NboStepInfo) -> c_int;
    // groups.rs:288 (GroupOptimizer::step after one unscale / clip decision over all gradients)
    pub fn nbo_fused_step_groups(n_groups: u64, opts: *const *mut NboOptim, params: *const *mut NboList,
                                 grads: *const *mut NboList, scaler: *mut NboScaler,
                                 all_grads: *mut NboList, max_norm: f64, flags: u32) -> c_int;
    // trainer.rs:253-267 (accumulation buffers: buf += g, optionally g = 0)
    pub fn nbo_accumulate(accum: *mut NboList, grads: *mut NboList, zero_grads: c_int) -> c_int;
    // trainer.rs:230-267 in one pass (scan + unscale + accumulate + the buffer's sum of squares;
    // flags: 1 = check finite without a scaler, 2 = write the unscaled gradients back), and
    // trainer.rs:274-290 over a buffer whose sum of squares is known
    pub fn nbo_unscale_accumulate(scaler: *mut NboScaler, accum: *mut NboList, grads: *mut NboList,
                                  flags: u32, ok: *mut c_int, accum_sumsq: *mut f64) -> c_int;
    pub fn nbo_fused_step_norm(opt: *mut NboOptim, params: *mut NboList, grads: *mut NboList,
                               max_norm: f64, sumsq: f64, flags: u32) -> c_int;
    pub fn nbo_fused_step_groups_norm(n_groups: u64, opts: *const *mut NboOptim, params: *const *mut NboList,
                                      grads: *const *mut NboList, max_norm: f64, sumsq: f64, flags: u32) -> c_int;
    // trainer.rs:387-400 (Trainer::has_non_finite)
    pub fn nbo_has_non_finite(grads: *mut NboList, found: *mut c_int) -> c_int;
    // nabla-core Backend primitives as multi-tensor launches (backend/mod.rs:82-216, 275-279):
    // op = 0 scale, 1 axpy_inplace, 2 add, 3 emul, 4 ediv, 5 powf, 6 map(x + s), 7 zeros, 8 clone
    pub fn nbo_backend_apply(op: c_int, out: *mut NboList, a: *mut NboList, b: *mut NboList, s: f64) -> c_int;
    pub fn nbo_backend_cast(dst: *mut NboList, src: *mut NboList) -> c_int;
    // checkpoint.rs:54-62, 92-99 over module/core.rs:66-120 (params.nbla / optim.nbla)
    pub fn nbo_nbla_save_list(path: *const c_char, list: *mut NboList, names: *const *const c_char) -> c_int;
    pub fn nbo_nbla_load_list(path: *const c_char, list: *mut NboList, names: *const *const c_char) -> c_int;
    pub fn nbo_optim_save_state(opt: *mut NboOptim, path: *const c_char) -> c_int;
    pub fn nbo_optim_load_state(opt: *mut NboOptim, path: *const c_char) -> c_int;
    // params.nbla of a mixed-precision optimizer: its f32 master weights (no counterpart in the reference)
    pub fn nbo_optim_save_master(opt: *mut NboOptim, path: *const c_char, names: *const *const c_char) -> c_int;
    pub fn nbo_optim_load_master(opt: *mut NboOptim, path: *const c_char, names: *const *const c_char) -> c_int;
    // groups.rs:320-350 (GroupOptimizer's state keys "g{gi}.m{i}" / "g{gi}.v{i}")
    pub fn nbo_optim_save_state_groups(n_groups: u64, opts: *const *mut NboOptim, path: *const c_char) -> c_int;
    pub fn nbo_optim_load_state_groups(n_groups: u64, opts: *const *mut NboOptim, path: *const c_char) -> c_int;
    // checkpoint.rs:54-58, 88-90 for a module whose parameters are spread over the groups
    pub fn nbo_optim_save_params_groups(n_groups: u64, opts: *const *mut NboOptim, params: *const *mut NboList,
                                        n_params: u64, group_of: *const u32, index_in_group: *const u32,
                                        names: *const *const c_char, path: *const c_char) -> c_int;
    pub fn nbo_optim_load_params_groups(n_groups: u64, opts: *const *mut NboOptim, params: *const *mut NboList,
                                        n_params: u64, group_of: *const u32, index_in_group: *const u32,
                                        names: *const *const c_char, path: *const c_char) -> c_int;
    pub fn nbo_optim_trace_read(opt: *mut NboOptim, out: *mut NboStepInfo, max_entries: u64,
                                n_out: *mut u64, total: *mut u64) -> c_int;
    pub fn nbo_optim_state_regions(opt: *mut NboOptim, regions: *mut c_int) -> c_int;
    pub fn nbo_optim_state_placement_note(opt: *mut NboOptim, buf: *mut c_char, buf_bytes: u64) -> c_int;
    pub fn nbo_status_string(status: c_int) -> *const c_char;
    pub fn nbo_version() -> *const c_char;
    // (measurement) the caller's tensors in named HBM regions
    pub fn nbo_alloc_placed(n_buffers: u32, bytes: u64, region: *const c_int, out_ptrs: *mut *mut c_void,
                            out: *mut *mut NboPlaced) -> c_int;
    pub fn nbo_free_placed(p: *mut NboPlaced) -> c_int;
    pub fn nbo_placed_note(p: *mut NboPlaced, buf: *mut c_char, buf_bytes: u64) -> c_int;
    // measurement helpers of nabla_optim_bench.h (no counterpart in the reference)
    pub fn nbo_copy_bytes(src_dev: *const c_void, dst_dev: *mut c_void, bytes: u64) -> c_int;
    pub fn nbo_hbm_ceiling(pattern: c_int, spread: c_int, bytes_per_stream: u64, reps: c_int, settle_ms: u32,
                           best_gbps: *mut f64, mean_gbps: *mut f64, regions: *mut c_int) -> c_int;
    pub fn nbo_hbm_ceiling_shape(pattern: c_int, shape: c_int, spread: c_int, bytes_per_stream: u64, reps: c_int,
                                 settle_ms: u32, best_gbps: *mut f64, mean_gbps: *mut f64, regions: *mut c_int,
                                 mismatches: *mut u64) -> c_int;
    pub fn nbo_hbm_ceiling_compare(pattern: c_int, n_shapes: c_int, shapes: *const c_int, iters: *const u32,
                                   spread: c_int, bytes_per_stream: u64, rounds: c_int, reps: c_int, settle_ms: u32,
                                   best_gbps: *mut f64, mean_gbps: *mut f64, regions: *mut c_int) -> c_int;
    pub fn nbo_selftest_half_arith(half_type: c_int, div_mismatches: *mut u64, sqrt_mismatches: *mut u64,
                                   example_pair: *mut u64, example_arg: *mut u64) -> c_int;
    pub fn nbo_profile_enable(on: c_int) -> c_int;
    pub fn nbo_profile_read(kernel_name: *const c_char, launches: *mut u64, total_ms: *mut f64) -> c_int;
}
