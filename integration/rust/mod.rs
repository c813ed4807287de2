//! `nabla-train/src/optim/mi355x/mod.rs` -- `Sgd` / `Adam` / `AdamW`, `GradScaler`, `clip_grad_norm`,
//! `zero_grad` and the fused Trainer tail on one MI355X, behind nabla-train's own
//! `Optimizer<T, B>` / `OptimState<T, B>` traits (`optim/core.rs:9-79`).
//!
//! UNVERIFIED SOURCE: the image this was written in has no Rust toolchain.  Signatures were
//! checked by eye against `nabla-train/src/optim/core.rs:9-79,254-260,334-413` and
//! `nabla-train/src/optim/alg.rs:20-105,181-252,319-381,471-671`; the C ABI underneath
//! (`ffi.rs`) is what is built and tested.
//!
//! Prerequisite in nabla-core: the HIP backend has to hand out its device addresses.
//! `BackendCore::device_ptr` exists (`common/backend/mod.rs:178-181`) but the HIP backend does
//! not override it (`cuda_hip/hip/backend.rs:470-514`), so it returns 0:
//!
//! ```ignore
//! // nabla-core/src/cuda_hip/hip/backend.rs, inside `impl BackendCore for Hip`
//! fn device_ptr<T: Scalar>(storage: &Self::Storage<T>) -> u64 { storage.buffer().ptr as u64 }
//! ```
//!
//! The reference's HIP backend launches on the null stream without syncing
//! (`hip/backend.rs:337,345-347`); so does this library by default, so its kernels order after
//! the backward pass that produced the gradients and before whatever reads the parameters next.

pub mod ffi;

use std::any::TypeId;
use std::cell::RefCell;
use std::collections::HashMap;
use std::ffi::{CStr, CString};
use std::marker::PhantomData;
use std::os::raw::{c_int, c_void};
use std::ptr;

use nabla_core::backend::Hip;
use nabla_core::scalar::Scalar;
use nabla_core::tensor::Tensor;

use crate::optim::core::{GradScalerState, OptimKind, OptimMeta, OptimState, Optimizer};

// ---- status codes -> the reference's panics and Err(String)s ------------------------------

fn last_error() -> String {
    unsafe { CStr::from_ptr(ffi::nbo_last_error()) }.to_string_lossy().into_owned()
}

/// Statuses 1..=3 carry the text of the reference's `assert_eq!` / shape panics
/// (`alg.rs:110-119`, `tensor/ops.rs:638-646`); anything else is a runtime failure, which the
/// reference's HIP backend also turns into a panic (`hip/backend.rs:342-344`).
fn check(rc: c_int) {
    if rc != ffi::NBO_OK {
        panic!("{}", last_error());
    }
}

/// Statuses 4..=6 are the reference's `Err(String)` of state loading (`alg.rs:487-516, 531-545`).
fn check_state(rc: c_int) -> Result<(), String> {
    if rc == ffi::NBO_OK {
        Ok(())
    } else {
        Err(last_error())
    }
}

/// Element type code of `T` (`f32`, `f64`, `half::bf16`, `half::f16`).
fn dtype_of<T: Scalar>() -> c_int {
    let t = TypeId::of::<T>();
    if t == TypeId::of::<f32>() {
        ffi::NBO_DT_F32
    } else if t == TypeId::of::<f64>() {
        ffi::NBO_DT_F64
    } else if t == TypeId::of::<half::bf16>() {
        ffi::NBO_DT_BF16
    } else if t == TypeId::of::<half::f16>() {
        ffi::NBO_DT_F16
    } else {
        panic!("nabla-train: mi355x optimizers support f32, f64, bf16 and f16 tensors")
    }
}

// ---- ListCache: a `&[&Tensor]` argument as an nbo_list, rebuilt only when it has to be ------

/// Keeps the `nbo_list` of the last call.  Same shapes and addresses: reused as it is.  Same
/// shapes, other addresses (fresh gradient tensors every step): only the address table is
/// uploaded again.  Anything else: a new list.
pub struct ListCache {
    h: *mut ffi::NboList,
    dtype: c_int,
    shapes: Vec<(usize, usize)>,
    ptrs: Vec<u64>,
}

impl ListCache {
    pub fn new() -> Self {
        Self { h: ptr::null_mut(), dtype: -1, shapes: Vec::new(), ptrs: Vec::new() }
    }

    pub fn get<T: Scalar>(&mut self, tensors: &[&Tensor<T, Hip>]) -> *mut ffi::NboList {
        let dtype = dtype_of::<T>();
        let shapes: Vec<(usize, usize)> = tensors.iter().map(|t| t.shape()).collect();
        let ptrs: Vec<u64> = tensors.iter().map(|t| t.device_ptr()).collect();
        if !self.h.is_null() && dtype == self.dtype && shapes == self.shapes {
            if ptrs != self.ptrs {
                let raw: Vec<*const c_void> = ptrs.iter().map(|&p| p as *const c_void).collect();
                check(unsafe { ffi::nbo_list_set_ptrs(self.h, raw.as_ptr()) });
                self.ptrs = ptrs;
            }
            return self.h;
        }
        self.release();
        let rows: Vec<u64> = shapes.iter().map(|s| s.0 as u64).collect();
        let cols: Vec<u64> = shapes.iter().map(|s| s.1 as u64).collect();
        let raw: Vec<*const c_void> = ptrs.iter().map(|&p| p as *const c_void).collect();
        let mut h: *mut ffi::NboList = ptr::null_mut();
        check(unsafe {
            ffi::nbo_list_create(shapes.len() as u64, rows.as_ptr(), cols.as_ptr(), dtype, raw.as_ptr(), &mut h)
        });
        self.h = h;
        self.dtype = dtype;
        self.shapes = shapes;
        self.ptrs = ptrs;
        h
    }

    fn release(&mut self) {
        if !self.h.is_null() {
            unsafe { ffi::nbo_list_destroy(self.h) };
            self.h = ptr::null_mut();
        }
    }
}

impl Default for ListCache {
    fn default() -> Self {
        Self::new()
    }
}

impl Drop for ListCache {
    fn drop(&mut self) {
        self.release();
    }
}

// ---- the engine handle shared by MiSgd / MiAdam / MiAdamW ------------------------------------

fn kind_code(kind: OptimKind) -> i32 {
    match kind {
        OptimKind::AdamW => ffi::NBO_KIND_ADAMW,
        OptimKind::Adam => ffi::NBO_KIND_ADAM,
        OptimKind::Sgd => ffi::NBO_KIND_SGD,
    }
}

fn to_nbo(meta: &OptimMeta) -> ffi::NboMeta {
    ffi::NboMeta {
        kind: kind_code(meta.kind),
        reserved: 0,
        lr: meta.lr,
        beta1: meta.beta1,
        beta2: meta.beta2,
        eps: meta.eps,
        weight_decay: meta.weight_decay,
        momentum: meta.momentum,
        step_count: meta.step_count as u64,
    }
}

/// Hyper-parameters as the builder setters leave them, and the library handle once the first
/// call needs it (the reference's constructors cannot fail and its builders run before any
/// step, so creation is deferred until the hyper-parameters are final).
struct Engine<T: Scalar> {
    meta: OptimMeta,
    shapes: Vec<(usize, usize)>,
    keep_master: bool,
    h: *mut ffi::NboOptim,
    params: ListCache,
    grads: ListCache,
    _t: PhantomData<T>,
}

impl<T: Scalar> Engine<T> {
    fn new(meta: OptimMeta, shapes: &[(usize, usize)], keep_master: bool) -> Self {
        Self {
            meta,
            shapes: shapes.to_vec(),
            keep_master,
            h: ptr::null_mut(),
            params: ListCache::new(),
            grads: ListCache::new(),
            _t: PhantomData,
        }
    }

    fn handle(&mut self) -> *mut ffi::NboOptim {
        if self.h.is_null() {
            let rows: Vec<u64> = self.shapes.iter().map(|s| s.0 as u64).collect();
            let cols: Vec<u64> = self.shapes.iter().map(|s| s.1 as u64).collect();
            let meta = to_nbo(&self.meta);
            // keep_master: bf16 / f16 tensors over f32 state; otherwise state and arithmetic are T
            let state_dtype = if self.keep_master { ffi::NBO_DT_F32 } else { dtype_of::<T>() };
            let mut h: *mut ffi::NboOptim = ptr::null_mut();
            check(unsafe {
                ffi::nbo_optim_create(&meta, self.shapes.len() as u64, rows.as_ptr(), cols.as_ptr(), state_dtype,
                                      self.keep_master as c_int, &mut h)
            });
            self.h = h;
        }
        self.h
    }

    fn step(&mut self, params: &mut [&mut Tensor<T, Hip>], grads: &[&Tensor<T, Hip>]) {
        let h = self.handle();
        let p_refs: Vec<&Tensor<T, Hip>> = params.iter().map(|p| &**p).collect();
        let p = self.params.get(&p_refs);
        let g = self.grads.get(grads);
        // the reference's length and shape asserts happen inside and come back as its panics
        check(unsafe { ffi::nbo_optim_step(h, p, g) });
    }

    fn reset(&mut self) {
        let h = self.handle();
        check(unsafe { ffi::nbo_optim_reset(h) });
    }

    fn set_lr(&mut self, lr: f64) {
        self.meta.lr = lr;
        if !self.h.is_null() {
            check(unsafe { ffi::nbo_optim_set_lr(self.h, lr) });
        }
    }

    /// step_count lives on the device (the skip decision of a fused step is taken there).
    fn step_count(&mut self) -> usize {
        if self.h.is_null() {
            return self.meta.step_count;
        }
        let mut m = to_nbo(&self.meta);
        check(unsafe { ffi::nbo_optim_get_meta(self.h, &mut m) });
        m.step_count as usize
    }

    /// One cloned state tensor, as `state_tensors()` returns them (`alg.rs:476-485`).
    fn read_state(&mut self, name: &str, shape: (usize, usize)) -> Tensor<T, Hip> {
        self.state_is_t();
        let h = self.handle();
        let t = Tensor::<T, Hip>::zeros(shape.0, shape.1);
        let key = CString::new(name).expect("state names hold no NUL");
        check(unsafe {
            ffi::nbo_optim_state_read(h, key.as_ptr(), t.device_ptr() as *mut c_void, (shape.0 * shape.1) as u64, 1)
        });
        t
    }

    fn write_state(&mut self, name: &str, t: &Tensor<T, Hip>) -> Result<(), String> {
        self.state_is_t();
        let h = self.handle();
        let key = CString::new(name).map_err(|_| format!("bad tensor key: {name}"))?;
        let (r, c) = t.shape();
        check_state(unsafe {
            ffi::nbo_optim_state_write(h, key.as_ptr(), t.device_ptr() as *const c_void, (r * c) as u64, 1)
        })
    }

    /// With f32 master weights the state is f32 whatever `T` is: a `Tensor<T, Hip>` cannot hold
    /// it, and the trait's `state_tensors` / `load_state_tensors` (typed in `T`) do not apply --
    /// `state_tensors_f32` / `load_state_tensors_f32` do.
    fn state_is_t(&self) {
        assert!(
            !self.keep_master || TypeId::of::<T>() == TypeId::of::<f32>(),
            "nabla-train: this optimizer keeps f32 state under 16-bit tensors; use state_tensors_f32 / load_state_tensors_f32"
        );
    }

    fn read_state_f32(&mut self, name: &str, shape: (usize, usize)) -> Tensor<f32, Hip> {
        assert!(self.keep_master, "f32 state access is for optimizers with f32 master weights");
        let h = self.handle();
        let t = Tensor::<f32, Hip>::zeros(shape.0, shape.1);
        let key = CString::new(name).expect("state names hold no NUL");
        check(unsafe {
            ffi::nbo_optim_state_read(h, key.as_ptr(), t.device_ptr() as *mut c_void, (shape.0 * shape.1) as u64, 1)
        });
        t
    }

    fn write_state_f32(&mut self, name: &str, t: &Tensor<f32, Hip>) -> Result<(), String> {
        assert!(self.keep_master, "f32 state access is for optimizers with f32 master weights");
        let h = self.handle();
        let key = CString::new(name).map_err(|_| format!("bad tensor key: {name}"))?;
        let (r, c) = t.shape();
        check_state(unsafe {
            ffi::nbo_optim_state_write(h, key.as_ptr(), t.device_ptr() as *const c_void, (r * c) as u64, 1)
        })
    }

    fn state_list(&mut self, prefixes: &[&str]) -> Vec<(String, Tensor<T, Hip>)> {
        let shapes = self.shapes.clone();
        let mut out = Vec::with_capacity(shapes.len() * prefixes.len());
        for prefix in prefixes {
            for (i, &s) in shapes.iter().enumerate() {
                let name = format!("{prefix}{i}");
                let t = self.read_state(&name, s);
                out.push((name, t));
            }
        }
        out
    }

    /// The key loop of `load_state_tensors` (`alg.rs:487-516, 564-593, 631-648`): it needs all
    /// names at once for "missing m{i}", so it stays on this side; nothing is written unless
    /// the whole list checks out.
    fn load_state_list(&mut self, tensors: &[(String, Tensor<T, Hip>)], prefixes: &[char]) -> Result<(), String> {
        let n = self.shapes.len();
        let mut slots: Vec<Vec<Option<&Tensor<T, Hip>>>> = prefixes.iter().map(|_| vec![None; n]).collect();
        for (name, t) in tensors {
            for (k, &prefix) in prefixes.iter().enumerate() {
                if let Some(idx) = name.strip_prefix(prefix) {
                    let i = idx.parse::<usize>().map_err(|_| format!("bad tensor key: {name}"))?;
                    if i >= n {
                        return Err(format!("{prefix} index out of range: {i}"));
                    }
                    slots[k][i] = Some(t);
                    break;
                }
            }
        }
        for (k, &prefix) in prefixes.iter().enumerate() {
            for i in 0..n {
                if slots[k][i].is_none() {
                    return Err(format!("missing {prefix}{i}"));
                }
            }
        }
        for (k, &prefix) in prefixes.iter().enumerate() {
            for i in 0..n {
                self.write_state(&format!("{prefix}{i}"), slots[k][i].unwrap())?;
            }
        }
        Ok(())
    }

    fn meta(&mut self) -> OptimMeta {
        if self.h.is_null() {
            return copy_meta(&self.meta);
        }
        let mut m = to_nbo(&self.meta);
        check(unsafe { ffi::nbo_optim_get_meta(self.h, &mut m) });
        OptimMeta {
            kind: self.meta.kind,
            lr: m.lr,
            beta1: m.beta1,
            beta2: m.beta2,
            eps: m.eps,
            weight_decay: m.weight_decay,
            momentum: m.momentum,
            step_count: m.step_count as usize,
        }
    }

    fn load_meta(&mut self, meta: &OptimMeta) -> Result<(), String> {
        if kind_code(meta.kind) != kind_code(self.meta.kind) {
            return Err("optim kind mismatch".to_owned());
        }
        let h = self.handle();
        check_state(unsafe { ffi::nbo_optim_load_meta(h, &to_nbo(meta)) })?;
        let kind = self.meta.kind;
        self.meta = copy_meta(meta);
        self.meta.kind = kind;
        Ok(())
    }
}

fn copy_meta(m: &OptimMeta) -> OptimMeta {
    OptimMeta {
        kind: m.kind,
        lr: m.lr,
        beta1: m.beta1,
        beta2: m.beta2,
        eps: m.eps,
        weight_decay: m.weight_decay,
        momentum: m.momentum,
        step_count: m.step_count,
    }
}

impl<T: Scalar> Drop for Engine<T> {
    fn drop(&mut self) {
        if !self.h.is_null() {
            unsafe { ffi::nbo_optim_destroy(self.h) };
        }
    }
}

// ---- AdamW (alg.rs:7-167, 471-546) -------------------------------------------------------------

pub struct MiAdamW<T: Scalar> {
    e: RefCell<Engine<T>>,
}

impl<T: Scalar> MiAdamW<T> {
    /// `AdamW::new` with its defaults (`alg.rs:20-39`).
    #[must_use]
    pub fn new(lr: f64, param_shapes: &[(usize, usize)]) -> Self {
        let meta = OptimMeta {
            kind: OptimKind::AdamW,
            lr,
            beta1: 0.9,
            beta2: 0.999,
            eps: 1e-8,
            weight_decay: 0.01,
            momentum: 0.0,
            step_count: 0,
        };
        Self { e: RefCell::new(Engine::new(meta, param_shapes, false)) }
    }

    #[must_use]
    pub fn from_params(lr: f64, params: &[&Tensor<T, Hip>]) -> Self {
        let shapes: Vec<(usize, usize)> = params.iter().map(|p| p.shape()).collect();
        Self::new(lr, &shapes)
    }

    /// No counterpart in the reference (its optimizers are generic in one `T`): bf16 / f16
    /// parameters and gradients over f32 master weights and moments.  Call before the first
    /// step; then `master_from_params` once.
    #[must_use]
    pub fn with_f32_master(mut self) -> Self {
        self.e.get_mut().keep_master = true;
        self
    }

    #[must_use]
    pub fn beta1(mut self, beta1: f64) -> Self {
        self.e.get_mut().meta.beta1 = beta1;
        self
    }

    #[must_use]
    pub fn beta2(mut self, beta2: f64) -> Self {
        self.e.get_mut().meta.beta2 = beta2;
        self
    }

    #[must_use]
    pub fn eps(mut self, eps: f64) -> Self {
        self.e.get_mut().meta.eps = eps;
        self
    }

    #[must_use]
    pub fn weight_decay(mut self, wd: f64) -> Self {
        self.e.get_mut().meta.weight_decay = wd;
        self
    }

    #[must_use]
    pub fn lr(&self) -> f64 {
        self.e.borrow().meta.lr
    }

    /// `&mut self`: the count is read from the device.
    pub fn step_count(&mut self) -> usize {
        self.e.get_mut().step_count()
    }

    /// Clones of the moments (the reference hands out slices of its own tensors, `alg.rs:81-88`;
    /// here the moments live in the engine's arena).
    pub fn moments(&mut self) -> (Vec<Tensor<T, Hip>>, Vec<Tensor<T, Hip>>) {
        let e = self.e.get_mut();
        let mut all = e.state_list(&["m", "v"]);
        let v = all.split_off(e.shapes.len());
        (all.into_iter().map(|x| x.1).collect(), v.into_iter().map(|x| x.1).collect())
    }

    pub fn set_state(&mut self, step_count: usize, beta1: f64, beta2: f64, eps: f64, weight_decay: f64, lr: f64) {
        let meta = OptimMeta {
            kind: OptimKind::AdamW,
            lr,
            beta1,
            beta2,
            eps,
            weight_decay,
            momentum: 0.0,
            step_count,
        };
        self.e.get_mut().load_meta(&meta).expect("same kind");
    }

    /// Moments and master weights of the mixed-precision composition, as f32 tensors under the
    /// keys `m{i}`, `v{i}`, `w{i}` (what a checkpoint of such an optimizer has to carry; the
    /// library also writes them to NBLA files itself, `nbo_optim_save_state` /
    /// `nbo_optim_save_master`).
    pub fn state_tensors_f32(&mut self) -> Vec<(String, Tensor<f32, Hip>)> {
        let e = self.e.get_mut();
        let shapes = e.shapes.clone();
        let mut out = Vec::with_capacity(3 * shapes.len());
        for prefix in ["m", "v", "w"] {
            for (i, &s) in shapes.iter().enumerate() {
                let name = format!("{prefix}{i}");
                let t = e.read_state_f32(&name, s);
                out.push((name, t));
            }
        }
        out
    }

    /// The reverse: every `m{i}`, `v{i}` and `w{i}` must be there (`missing m{i}` otherwise, as
    /// `alg.rs:487-516` says it); afterwards the master weights count as set.
    pub fn load_state_tensors_f32(&mut self, tensors: &[(String, Tensor<f32, Hip>)]) -> Result<(), String> {
        let e = self.e.get_mut();
        let n = e.shapes.len();
        for prefix in ["m", "v", "w"] {
            for i in 0..n {
                let key = format!("{prefix}{i}");
                if !tensors.iter().any(|(name, _)| *name == key) {
                    return Err(format!("missing {key}"));
                }
            }
        }
        for (name, t) in tensors {
            e.write_state_f32(name, t)?; // bad keys and indices come back as the reference's errors
        }
        Ok(())
    }

    /// master = f32(params), for the mixed-precision composition.
    pub fn master_from_params(&mut self, params: &[&Tensor<T, Hip>]) {
        let e = self.e.get_mut();
        let h = e.handle();
        let p = e.params.get(params);
        check(unsafe { ffi::nbo_optim_master_from_params(h, p) });
    }

    /// The Trainer's tail after backward (`trainer.rs:230-291`) in three launches: unscale +
    /// found-inf + loss-scale update, clip, step, optional zeroing of the gradients; a
    /// non-finite gradient skips the step on the device.  Nothing is read back; `last_step`
    /// tells what was decided.  A skipped step leaves zeros in the gradients, as
    /// `GradScaler::unscale_and_update` does (`optim/core.rs:372-375`).
    pub fn fused_step(&mut self, scaler: Option<&mut MiGradScaler>, params: &mut [&mut Tensor<T, Hip>],
                      grads: &[&Tensor<T, Hip>], max_norm: f64, zero_grads: bool) {
        let e = self.e.get_mut();
        let h = e.handle();
        let p_refs: Vec<&Tensor<T, Hip>> = params.iter().map(|p| &**p).collect();
        let p = e.params.get(&p_refs);
        let g = e.grads.get(grads);
        let s = scaler.map_or(ptr::null_mut(), |s| s.h);
        let flags = ffi::NBO_STEP_ZERO_ON_SKIP | if zero_grads { ffi::NBO_STEP_ZERO_GRADS } else { 0 };
        check(unsafe { ffi::nbo_fused_step(h, s, p, g, max_norm, flags) });
    }

    pub fn last_step(&mut self) -> ffi::NboStepInfo {
        let h = self.e.get_mut().handle();
        let mut info = ffi::NboStepInfo { scale: 0.0, norm: 0.0, step_count: 0, found_inf: 0, clipped: 0 };
        check(unsafe { ffi::nbo_optim_last_step(h, &mut info) });
        info
    }
}

impl<T: Scalar> Optimizer<T, Hip> for MiAdamW<T> {
    fn step(&mut self, params: &mut [&mut Tensor<T, Hip>], grads: &[&Tensor<T, Hip>]) {
        self.e.get_mut().step(params, grads);
    }
    fn reset(&mut self) {
        self.e.get_mut().reset();
    }
    fn set_lr(&mut self, lr: f64) {
        self.e.get_mut().set_lr(lr);
    }
}

// `OptimState` takes `&self` for `state_tensors` and `meta`, while the engine creates its handle
// lazily and reads through it: hence the `RefCell` around it.
impl<T: Scalar> OptimState<T, Hip> for MiAdamW<T> {
    fn kind(&self) -> OptimKind {
        OptimKind::AdamW
    }
    fn state_tensors(&self) -> Vec<(String, Tensor<T, Hip>)> {
        self.e.borrow_mut().state_list(&["m", "v"])
    }
    fn load_state_tensors(&mut self, tensors: &[(String, Tensor<T, Hip>)]) -> Result<(), String> {
        self.e.get_mut().load_state_list(tensors, &['m', 'v'])
    }
    fn meta(&self) -> OptimMeta {
        // AdamW::meta reports momentum 0 (alg.rs:518-529)
        self.e.borrow_mut().meta()
    }
    fn load_meta(&mut self, meta: &OptimMeta) -> Result<(), String> {
        self.e.get_mut().load_meta(meta)
    }
}

// ---- Adam (alg.rs:169-308, 548-616) --------------------------------------------------------------

pub struct MiAdam<T: Scalar> {
    e: RefCell<Engine<T>>,
}

impl<T: Scalar> MiAdam<T> {
    /// `Adam::new` with its defaults (`alg.rs:181-199`).
    #[must_use]
    pub fn new(lr: f64, param_shapes: &[(usize, usize)]) -> Self {
        let meta = OptimMeta {
            kind: OptimKind::Adam,
            lr,
            beta1: 0.9,
            beta2: 0.999,
            eps: 1e-8,
            weight_decay: 0.0,
            momentum: 0.0,
            step_count: 0,
        };
        Self { e: RefCell::new(Engine::new(meta, param_shapes, false)) }
    }

    #[must_use]
    pub fn from_params(lr: f64, params: &[&Tensor<T, Hip>]) -> Self {
        let shapes: Vec<(usize, usize)> = params.iter().map(|p| p.shape()).collect();
        Self::new(lr, &shapes)
    }

    #[must_use]
    pub fn beta1(mut self, beta1: f64) -> Self {
        self.e.get_mut().meta.beta1 = beta1;
        self
    }

    #[must_use]
    pub fn beta2(mut self, beta2: f64) -> Self {
        self.e.get_mut().meta.beta2 = beta2;
        self
    }

    #[must_use]
    pub fn eps(mut self, eps: f64) -> Self {
        self.e.get_mut().meta.eps = eps;
        self
    }

    #[must_use]
    pub fn lr(&self) -> f64 {
        self.e.borrow().meta.lr
    }

    pub fn step_count(&mut self) -> usize {
        self.e.get_mut().step_count()
    }

    pub fn moments(&mut self) -> (Vec<Tensor<T, Hip>>, Vec<Tensor<T, Hip>>) {
        let e = self.e.get_mut();
        let mut all = e.state_list(&["m", "v"]);
        let v = all.split_off(e.shapes.len());
        (all.into_iter().map(|x| x.1).collect(), v.into_iter().map(|x| x.1).collect())
    }

    pub fn set_state(&mut self, step_count: usize, beta1: f64, beta2: f64, eps: f64, lr: f64) {
        let meta = OptimMeta {
            kind: OptimKind::Adam,
            lr,
            beta1,
            beta2,
            eps,
            weight_decay: 0.0,
            momentum: 0.0,
            step_count,
        };
        self.e.get_mut().load_meta(&meta).expect("same kind");
    }
}

impl<T: Scalar> Optimizer<T, Hip> for MiAdam<T> {
    fn step(&mut self, params: &mut [&mut Tensor<T, Hip>], grads: &[&Tensor<T, Hip>]) {
        self.e.get_mut().step(params, grads);
    }
    fn reset(&mut self) {
        self.e.get_mut().reset();
    }
    fn set_lr(&mut self, lr: f64) {
        self.e.get_mut().set_lr(lr);
    }
}

impl<T: Scalar> OptimState<T, Hip> for MiAdam<T> {
    fn kind(&self) -> OptimKind {
        OptimKind::Adam
    }
    fn state_tensors(&self) -> Vec<(String, Tensor<T, Hip>)> {
        self.e.borrow_mut().state_list(&["m", "v"])
    }
    fn load_state_tensors(&mut self, tensors: &[(String, Tensor<T, Hip>)]) -> Result<(), String> {
        self.e.get_mut().load_state_list(tensors, &['m', 'v'])
    }
    fn meta(&self) -> OptimMeta {
        self.e.borrow_mut().meta()
    }
    fn load_meta(&mut self, meta: &OptimMeta) -> Result<(), String> {
        self.e.get_mut().load_meta(meta)
    }
}

// ---- Sgd (alg.rs:310-428, 618-671) -----------------------------------------------------------------

pub struct MiSgd<T: Scalar> {
    e: RefCell<Engine<T>>,
}

impl<T: Scalar> MiSgd<T> {
    /// `Sgd::new` with its defaults (`alg.rs:319-330`).
    #[must_use]
    pub fn new(lr: f64, param_shapes: &[(usize, usize)]) -> Self {
        let meta = OptimMeta {
            kind: OptimKind::Sgd,
            lr,
            beta1: 0.0,
            beta2: 0.0,
            eps: 0.0,
            weight_decay: 0.0,
            momentum: 0.0,
            step_count: 0,
        };
        Self { e: RefCell::new(Engine::new(meta, param_shapes, false)) }
    }

    #[must_use]
    pub fn from_params(lr: f64, params: &[&Tensor<T, Hip>]) -> Self {
        let shapes: Vec<(usize, usize)> = params.iter().map(|p| p.shape()).collect();
        Self::new(lr, &shapes)
    }

    #[must_use]
    pub fn momentum(mut self, momentum: f64) -> Self {
        self.e.get_mut().meta.momentum = momentum;
        self
    }

    #[must_use]
    pub fn weight_decay(mut self, wd: f64) -> Self {
        self.e.get_mut().meta.weight_decay = wd;
        self
    }

    #[must_use]
    pub fn lr(&self) -> f64 {
        self.e.borrow().meta.lr
    }

    #[must_use]
    pub fn momentum_value(&self) -> f64 {
        self.e.borrow().meta.momentum
    }

    #[must_use]
    pub fn weight_decay_value(&self) -> f64 {
        self.e.borrow().meta.weight_decay
    }

    /// Clones of the velocity tensors (`alg.rs:365-372` hands out slices of its own).
    pub fn velocity(&mut self) -> Vec<Tensor<T, Hip>> {
        self.e.get_mut().state_list(&["v"]).into_iter().map(|x| x.1).collect()
    }

    pub fn set_state(&mut self, lr: f64, momentum: f64, weight_decay: f64) {
        let meta = OptimMeta {
            kind: OptimKind::Sgd,
            lr,
            beta1: 0.0,
            beta2: 0.0,
            eps: 0.0,
            weight_decay,
            momentum,
            step_count: 0,
        };
        self.e.get_mut().load_meta(&meta).expect("same kind");
    }
}

impl<T: Scalar> Optimizer<T, Hip> for MiSgd<T> {
    fn step(&mut self, params: &mut [&mut Tensor<T, Hip>], grads: &[&Tensor<T, Hip>]) {
        self.e.get_mut().step(params, grads);
    }
    fn reset(&mut self) {
        self.e.get_mut().reset();
    }
    fn set_lr(&mut self, lr: f64) {
        self.e.get_mut().set_lr(lr);
    }
}

impl<T: Scalar> OptimState<T, Hip> for MiSgd<T> {
    fn kind(&self) -> OptimKind {
        OptimKind::Sgd
    }
    fn state_tensors(&self) -> Vec<(String, Tensor<T, Hip>)> {
        self.e.borrow_mut().state_list(&["v"]) // velocity under "v{i}" (alg.rs:623-629)
    }
    fn load_state_tensors(&mut self, tensors: &[(String, Tensor<T, Hip>)]) -> Result<(), String> {
        self.e.get_mut().load_state_list(tensors, &['v'])
    }
    fn meta(&self) -> OptimMeta {
        self.e.borrow_mut().meta()
    }
    fn load_meta(&mut self, meta: &OptimMeta) -> Result<(), String> {
        self.e.get_mut().load_meta(meta)
    }
}

// ---- GradScaler (optim/core.rs:254-260, 334-413) ------------------------------------------------------

/// The loss scale, its factors and counters live on the device: the fused step updates them
/// there.  `state()` / `scale_factor()` read them back.
pub struct MiGradScaler {
    h: *mut ffi::NboScaler,
    grads: ListCache,
}

impl MiGradScaler {
    /// `GradScaler::new` (`core.rs:336-344`): scale 65536, growth 2, backoff 0.5, interval 2000.
    #[must_use]
    pub fn new() -> Self {
        let mut h: *mut ffi::NboScaler = ptr::null_mut();
        check(unsafe { ffi::nbo_scaler_create(ptr::null(), &mut h) });
        Self { h, grads: ListCache::new() }
    }

    #[must_use]
    pub fn scale_loss<T: Scalar>(&self, loss: &Tensor<T, Hip>) -> Tensor<T, Hip> {
        loss * T::from_f64(self.scale_factor()) // core.rs:347-349
    }

    /// `core.rs:351-388`: in place, in the gradients' own type; `false` on inf / NaN (the
    /// gradients are then zeros and the scale backed off).
    pub fn unscale_and_update<T: Scalar>(&mut self, grads: &mut [Tensor<T, Hip>]) -> bool {
        let refs: Vec<&Tensor<T, Hip>> = grads.iter().collect();
        let g = self.grads.get(&refs);
        let mut ok: c_int = 0;
        check(unsafe { ffi::nbo_scaler_unscale_and_update(self.h, g, &mut ok) });
        ok != 0
    }

    #[must_use]
    pub fn scale_factor(&self) -> f64 {
        self.state().scale
    }

    #[must_use]
    pub fn state(&self) -> GradScalerState {
        let mut s = ffi::NboScalerState {
            scale: 0.0,
            growth_factor: 0.0,
            backoff_factor: 0.0,
            growth_interval: 0,
            consecutive_ok: 0,
        };
        check(unsafe { ffi::nbo_scaler_state_get(self.h, &mut s) });
        GradScalerState {
            scale: s.scale,
            growth_factor: s.growth_factor,
            backoff_factor: s.backoff_factor,
            growth_interval: s.growth_interval as usize,
            consecutive_ok: s.consecutive_ok as usize,
        }
    }

    pub fn load_state(&mut self, state: &GradScalerState) {
        let s = ffi::NboScalerState {
            scale: state.scale,
            growth_factor: state.growth_factor,
            backoff_factor: state.backoff_factor,
            growth_interval: state.growth_interval as u64,
            consecutive_ok: state.consecutive_ok as u64,
        };
        check(unsafe { ffi::nbo_scaler_load_state(self.h, &s) });
    }
}

impl Default for MiGradScaler {
    fn default() -> Self {
        Self::new()
    }
}

impl Drop for MiGradScaler {
    fn drop(&mut self) {
        unsafe { ffi::nbo_scaler_destroy(self.h) };
    }
}

// ---- free functions ----------------------------------------------------------------------------------

thread_local! {
    static FREE_LISTS: std::cell::RefCell<HashMap<&'static str, ListCache>> = std::cell::RefCell::new(HashMap::new());
}

fn with_list<T: Scalar, R>(slot: &'static str, tensors: &[&Tensor<T, Hip>], f: impl FnOnce(*mut ffi::NboList) -> R) -> R {
    FREE_LISTS.with(|m| {
        let mut m = m.borrow_mut();
        let h = m.entry(slot).or_insert_with(ListCache::new).get(tensors);
        f(h)
    })
}

/// `clip_grad_norm` (`nabla-train/src/trainer.rs:500-523`): returns the pre-clip norm, 0 when
/// `max_norm <= 0`.
pub fn clip_grad_norm<T: Scalar>(grads: &mut [Tensor<T, Hip>], max_norm: f64) -> f64 {
    let refs: Vec<&Tensor<T, Hip>> = grads.iter().collect();
    with_list("clip", &refs, |g| {
        let mut norm = 0.0f64;
        check(unsafe { ffi::nbo_clip_grad_norm(g, max_norm, &mut norm) });
        norm
    })
}

/// `zero_grad` (`nabla-ml/src/autograd/ops.rs:1668-1673`) over gradient tensors.
pub fn zero_grad<T: Scalar>(grads: &mut [Tensor<T, Hip>]) {
    let refs: Vec<&Tensor<T, Hip>> = grads.iter().collect();
    with_list("zero", &refs, |g| check(unsafe { ffi::nbo_zero_grad(g) }));
}

/// `scale_grad` (`autograd/ops.rs:1675-1680`).
pub fn scale_grad<T: Scalar>(grads: &mut [Tensor<T, Hip>], factor: f64) {
    let refs: Vec<&Tensor<T, Hip>> = grads.iter().collect();
    with_list("scale", &refs, |g| check(unsafe { ffi::nbo_scale_grad(g, factor) }));
}

/// `Trainer::has_non_finite` (`trainer.rs:387-400`).
pub fn has_non_finite<T: Scalar>(grads: &[Tensor<T, Hip>]) -> bool {
    let refs: Vec<&Tensor<T, Hip>> = grads.iter().collect();
    with_list("finite", &refs, |g| {
        let mut found: c_int = 0;
        check(unsafe { ffi::nbo_has_non_finite(g, &mut found) });
        found != 0
    })
}

/// The free function `adamw_step` (`alg.rs:431-469`): one tensor, caller-held moments.  The
/// engine owns its moments, so this writes the caller's into a one-tensor optimizer at
/// `step - 1`, steps once and reads them back.
#[allow(clippy::too_many_arguments)]
pub fn adamw_step<T: Scalar>(param: &mut Tensor<T, Hip>, grad: &Tensor<T, Hip>, m: &mut Tensor<T, Hip>,
                             v: &mut Tensor<T, Hip>, lr: f64, beta1: f64, beta2: f64, eps: f64, weight_decay: f64,
                             step: usize) {
    let mut opt = MiAdamW::<T>::new(lr, &[param.shape()]).beta1(beta1).beta2(beta2).eps(eps).weight_decay(weight_decay);
    let e = opt.e.get_mut();
    e.meta.step_count = step.saturating_sub(1);
    e.write_state("m0", m).expect("m0");
    e.write_state("v0", v).expect("v0");
    e.step(&mut [param], &[grad]);
    *m = e.read_state("m0", m.shape());
    *v = e.read_state("v0", v.shape());
}

/// `B::sync` for this library's stream.
pub fn sync() {
    check(unsafe { ffi::nbo_sync() });
}
