//! MI355X backend of tur's quantized linear layers, over `libturq` (turq-sys).
//!
//! What tur binds: `HipDevice` (the `Device` handed to `QVarBuilder::from_gguf`, src/weights/gguf_varbuilder.rs:20-30),
//! `HipQVarBuilder::get / get_no_shape` (gguf_varbuilder.rs:52-94), `HipQTensor` (`Arc<QTensor>`), `HipQMatMul` with candle's
//! `QMatMul::forward` contract (src/models/layers/linear.rs:19-31), and `HipRmsNorm` (src/models/layers/norm.rs:52-94).
//! The `LinearX::Hip` arm that uses them is at the end of this file as the patch against src/models/layers/linear.rs.
//!
//! UNCOMPILED in the tree this file ships in (no Rust toolchain there).  The same calls, in the same order, are exercised
//! through the C++ mirror (tur_amd/csrc/host/turq.hpp, tests/cpp/test_host.cpp) and the ctypes mirror (tur_amd/qlinear.py).
//!
//! Errors are `candle_core::Error::Msg` with the text of `turq_last_error`, so they surface as `TurError::CandleError`
//! (src/shared/errors.rs:5-6); nothing here unwraps, expects or panics (the project's lints deny them, Cargo.toml:80-86).
//! Threading: a `HipDevice` is one context = one stream, and libturq contexts are thread-compatible, not thread-safe (a call may
//! grow or swap the context's scratch buffers under another call's feet).  The context therefore sits behind a `Mutex`: clones
//! of a `HipDevice` may live on several threads, as candle's `Device` may, and every call holds the lock for its duration.  tur
//! itself drives a model from one worker thread (src/server/worker.rs:69-100), so the lock is uncontended there.  Weights are
//! immutable after upload and reference counted.

use std::ffi::{CStr, CString};
use std::os::raw::{c_int, c_void};
use std::ptr;
use std::sync::{Arc, Mutex, MutexGuard};

use candle_core::{Device, Error, Result, Tensor};
use turq_sys::*;

fn fail(ctx: *const turq_ctx) -> Error {
    // SAFETY: turq_last_error returns a NUL-terminated string owned by the context (or by the thread when ctx is null)
    let msg = unsafe { CStr::from_ptr(turq_last_error(ctx)) }.to_string_lossy().into_owned();
    Error::Msg(msg)
}

fn check(ctx: *const turq_ctx, rc: c_int) -> Result<()> {
    if rc == TURQ_OK {
        Ok(())
    } else {
        Err(fail(ctx))
    }
}

struct Ctx(*mut turq_ctx);
// SAFETY: a context may be created on one thread and used on another, one thread at a time: it is only reachable through the
// Mutex of HipDevice (Send, deliberately NOT Sync: nothing in libturq locks a context)
unsafe impl Send for Ctx {}
impl Drop for Ctx {
    fn drop(&mut self) {
        // SAFETY: the pointer came from turq_ctx_create and is dropped once
        unsafe { turq_ctx_destroy(self.0) }
    }
}

/// One GPU context: device ordinal, stream, scratch.  Cheap to clone; calls through any clone are serialised by the lock.
#[derive(Clone)]
pub struct HipDevice(Arc<Mutex<Ctx>>);

impl HipDevice {
    /// the device picked where src/main.rs:188 / src/bin/server.rs:112 pick Metal or CPU today
    pub fn new(ordinal: usize) -> Result<Self> {
        let mut ctx = ptr::null_mut();
        // SAFETY: `ctx` is a valid out pointer
        check(ptr::null(), unsafe { turq_ctx_create(ordinal as c_int, &mut ctx) })?;
        Ok(Self(Arc::new(Mutex::new(Ctx(ctx)))))
    }
    /// the context, locked for the caller's scope (`guard.0` is the raw pointer)
    fn lock(&self) -> Result<MutexGuard<'_, Ctx>> {
        self.0.lock().map_err(|_| Error::Msg("the turq context's lock is poisoned (a call panicked while holding it)".into()))
    }
    pub fn synchronize(&self) -> Result<()> {
        let guard = self.lock()?;
        // SAFETY: the context is alive as long as `self`
        check(guard.0, unsafe { turq_sync(guard.0) })
    }
    /// Activations of any finite f32 magnitude on device pointers (host tensors always get them): see turq.h
    pub fn set_wide_activations(&self, on: bool) -> Result<()> {
        let guard = self.lock()?;
        // SAFETY: the context is alive
        check(guard.0, unsafe { turq_ctx_set_wide_activations(guard.0, on as c_int) })
    }
    /// Results stored since the last reset that were no finite numbers (an input left the f16 range, or was an infinity / NaN)
    pub fn nonfinite_count(&self, reset: bool) -> Result<u64> {
        let guard = self.lock()?;
        let mut n = 0u64;
        // SAFETY: `n` is a valid out pointer
        check(guard.0, unsafe { turq_ctx_nonfinite_count(guard.0, &mut n, reset as c_int) })?;
        Ok(n)
    }
}

/// `Arc<QTensor>` on the GPU: raw GGUF blocks of an (n, k) tensor in HBM, shared by its clones.
pub struct HipQTensor {
    dev: HipDevice,
    w: *mut turq_weight,
    dtype: c_int,
    n: usize,
    k: usize,
    one_dim: bool,
}
// SAFETY: the device copy is immutable after upload and its reference count is atomic
unsafe impl Send for HipQTensor {}
unsafe impl Sync for HipQTensor {}

impl Clone for HipQTensor {
    fn clone(&self) -> Self {
        // SAFETY: `w` is alive; retain cannot fail on a non-null handle
        unsafe { turq_weight_retain(self.w) };
        Self { dev: self.dev.clone(), w: self.w, dtype: self.dtype, n: self.n, k: self.k, one_dim: self.one_dim }
    }
}
impl Drop for HipQTensor {
    fn drop(&mut self) {
        // SAFETY: one release per handle held
        unsafe { turq_weight_release(self.w) };
    }
}

impl HipQTensor {
    fn from_handle(dev: &HipDevice, w: *mut turq_weight, one_dim: bool) -> Result<Self> {
        let (mut dtype, mut n, mut k) = (0 as c_int, 0i64, 0i64);
        // SAFETY: out pointers are valid; unused ones may be null (no context is involved: the error text is the thread's)
        check(ptr::null(), unsafe { turq_weight_info(w, &mut dtype, &mut n, &mut k, ptr::null_mut(), ptr::null_mut()) })?;
        Ok(Self { dev: dev.clone(), w, dtype, n: n as usize, k: k as usize, one_dim })
    }
    /// raw GGUF block bytes of a tensor of shape (n, k); quantized tensors go to the tiled layout the matmul kernels read
    pub fn from_blocks(dev: &HipDevice, ggml_dtype: u32, n: usize, k: usize, bytes: &[u8]) -> Result<Self> {
        let dt = ggml_dtype as c_int;
        let quant = matches!(dt, TURQ_Q8_0 | TURQ_Q4_K | TURQ_Q5_K | TURQ_Q6_K);
        let layout = if quant { TURQ_LAYOUT_TILED } else { TURQ_LAYOUT_NATIVE };
        let mut w = ptr::null_mut();
        {
            let guard = dev.lock()?;
            // SAFETY: `bytes` outlives the call, which copies them
            check(guard.0, unsafe {
                turq_weight_upload(guard.0, dt, n as i64, k as i64, bytes.as_ptr().cast(), bytes.len(), layout, &mut w)
            })?;
        }
        Self::from_handle(dev, w, false)
    }
    pub fn shape(&self) -> Vec<usize> {
        if self.one_dim {
            vec![self.k]
        } else {
            vec![self.n, self.k]
        }
    }
    pub fn ggml_dtype(&self) -> u32 {
        self.dtype as u32
    }
    /// `QTensor::dequantize(device)`: the f32 tensor, bit-exact with candle's `to_float`
    pub fn dequantize(&self, device: &Device) -> Result<Tensor> {
        let mut out = vec![0f32; self.n * self.k];
        {
            let guard = self.dev.lock()?;
            // SAFETY: `out` holds n * k floats
            check(guard.0, unsafe { turq_dequantize(guard.0, self.w, out.as_mut_ptr(), TURQ_MEM_HOST) })?;
        }
        Tensor::from_vec(out, self.shape(), device)
    }
    /// A hint that this weight belongs to one of the next forward calls (see turq_weight_prefetch: a read-only pass next to
    /// whatever the device runs; results are unaffected)
    pub fn prefetch(&self) -> Result<()> {
        let guard = self.dev.lock()?;
        // SAFETY: the weight and the context are alive
        check(guard.0, unsafe { turq_weight_prefetch(guard.0, self.w) })
    }
}

/// `QMatMul::from_arc(qtensor)` + `forward`, with candle's contract: rank >= 2, last dim == k, contiguous, f32 in, f32 out.
#[derive(Clone)]
pub struct HipQMatMul {
    t: HipQTensor,
    dense: bool,
}

fn rows_of(xs: &Tensor, k: usize) -> Result<(usize, Vec<usize>)> {
    let dims = xs.dims().to_vec();
    if dims.len() < 2 || dims[dims.len() - 1] != k {
        candle_core::bail!("shape mismatch in matmul: input {:?}, weight needs last dim {}", dims, k)
    }
    if !xs.is_contiguous() {
        candle_core::bail!("QMatMul::forward needs a contiguous input")
    }
    let m = dims[..dims.len() - 1].iter().product();
    Ok((m, dims))
}

impl HipQMatMul {
    /// block-quantized tensors give the quantized matmul; F32 / F16 / BF16 tensors (and every tensor while
    /// CANDLE_DEQUANTIZE_ALL is set) the dense one, as in candle
    pub fn from_arc(t: HipQTensor) -> Result<Self> {
        let quant = matches!(t.dtype, TURQ_Q8_0 | TURQ_Q4_K | TURQ_Q5_K | TURQ_Q6_K);
        let all = std::env::var_os("CANDLE_DEQUANTIZE_ALL").is_some() || std::env::var_os("CANDLE_DEQUANTIZE_ALL_F16").is_some();
        if quant && all {
            // the dense arm reads GGUF byte order: export the tiled copy and upload it once more as it is in the file
            let nbytes = unsafe { turq_weight_nbytes(t.dtype, t.n as i64, t.k as i64) };
            let mut raw = vec![0u8; nbytes];
            let mut w = ptr::null_mut();
            {
                let guard = t.dev.lock()?;
                // SAFETY: `raw` holds the tensor's GGUF size
                check(guard.0, unsafe { turq_weight_export(guard.0, t.w, raw.as_mut_ptr().cast(), nbytes) })?;
                check(guard.0, unsafe {
                    turq_weight_upload(guard.0, t.dtype, t.n as i64, t.k as i64, raw.as_ptr().cast(), nbytes, TURQ_LAYOUT_NATIVE, &mut w)
                })?;
            }
            return Ok(Self { t: HipQTensor::from_handle(&t.dev, w, false)?, dense: true });
        }
        Ok(Self { t, dense: !quant })
    }

    /// While candle has no HIP tensor type the activations are host tensors: TURQ_MEM_HOST stages them through the context.
    pub fn forward(&self, xs: &Tensor) -> Result<Tensor> {
        let (n, k) = (self.t.n, self.t.k);
        let (m, mut dims) = rows_of(xs, k)?;
        let x: Vec<f32> = xs.flatten_all()?.to_vec1()?;
        let mut y = vec![0f32; m * n];
        let algo = if self.dense { TURQ_ALGO_SIMPLE } else { TURQ_ALGO_AUTO };
        let guard = self.t.dev.lock()?;
        let ctx = guard.0;
        // SAFETY: x holds m * k floats, y m * n
        check(ctx, unsafe {
            turq_qmatmul(ctx, self.t.w, x.as_ptr().cast(), TURQ_ACT_F32, m as i64, k as i64, y.as_mut_ptr().cast(), TURQ_ACT_F32, n as i64,
                         ptr::null(), TURQ_MEM_HOST, algo)
        })?;
        if let Some(last) = dims.last_mut() {
            *last = n;
        }
        Tensor::from_vec(y, dims, xs.device())
    }

    /// `residual + forward(xs)`: the residual connection (`x + h`, src/models/qwen3.rs:635) taken into the matmul's store
    /// (TURQ_OUT_ACCUMULATE); `residual` has the output's shape.
    pub fn forward_add(&self, xs: &Tensor, residual: &Tensor) -> Result<Tensor> {
        let (n, k) = (self.t.n, self.t.k);
        let (m, mut dims) = rows_of(xs, k)?;
        let x: Vec<f32> = xs.flatten_all()?.to_vec1()?;
        let mut y: Vec<f32> = residual.flatten_all()?.to_vec1()?;
        if y.len() != m * n {
            candle_core::bail!("shape mismatch in matmul: the residual has {} elements, the output {}", y.len(), m * n)
        }
        let algo = if self.dense { TURQ_ALGO_SIMPLE } else { TURQ_ALGO_AUTO };
        let guard = self.t.dev.lock()?;
        let ctx = guard.0;
        // SAFETY: x holds m * k floats, y m * n
        check(ctx, unsafe {
            turq_qmatmul(ctx, self.t.w, x.as_ptr().cast(), TURQ_ACT_F32, m as i64, k as i64, y.as_mut_ptr().cast(),
                         TURQ_ACT_F32 | TURQ_OUT_ACCUMULATE, n as i64, ptr::null(), TURQ_MEM_HOST, algo)
        })?;
        if let Some(last) = dims.last_mut() {
            *last = n;
        }
        Tensor::from_vec(y, dims, xs.device())
    }

    /// The projections the reference calls back to back on one tensor - q / k / v (src/models/qwen3.rs:272-274), gate / up
    /// (src/models/qwen3.rs:161-167) - in one call: with device-resident activations one kernel launch per run of equal formats.
    pub fn forward_multi(layers: &[&HipQMatMul], xs: &Tensor) -> Result<Vec<Tensor>> {
        let Some(first) = layers.first() else { return Ok(Vec::new()) };
        let k = first.t.k;
        let (m, dims) = rows_of(xs, k)?;
        if layers.iter().any(|l| l.t.k != k || l.dense) {
            return layers.iter().map(|l| l.forward(xs)).collect();
        }
        let x: Vec<f32> = xs.flatten_all()?.to_vec1()?;
        let mut ys: Vec<Vec<f32>> = layers.iter().map(|l| vec![0f32; m * l.t.n]).collect();
        let ws: Vec<*const turq_weight> = layers.iter().map(|l| l.t.w as *const turq_weight).collect();
        let yp: Vec<*mut c_void> = ys.iter_mut().map(|y| y.as_mut_ptr().cast()).collect();
        let ld: Vec<i64> = layers.iter().map(|l| l.t.n as i64).collect();
        let guard = first.t.dev.lock()?;
        let ctx = guard.0;
        // SAFETY: the arrays have one entry per layer and every buffer its full size
        check(ctx, unsafe {
            turq_qmatmul_multi(ctx, ws.len() as c_int, ws.as_ptr(), x.as_ptr().cast(), TURQ_ACT_F32, m as i64, k as i64, yp.as_ptr(),
                               TURQ_ACT_F32, ld.as_ptr(), ptr::null(), TURQ_MEM_HOST, TURQ_ALGO_AUTO)
        })?;
        ys.into_iter()
            .zip(layers)
            .map(|(y, l)| {
                let mut d = dims.clone();
                if let Some(last) = d.last_mut() {
                    *last = l.t.n;
                }
                Tensor::from_vec(y, d, xs.device())
            })
            .collect()
    }

    /// `act_fn(gate_proj(x)) * up_proj(x)`, the first half of `Qwen3MLP::forward` (src/models/qwen3.rs:161-167), SiLU.
    pub fn forward_gate_up(gate: &HipQMatMul, up: &HipQMatMul, xs: &Tensor) -> Result<Tensor> {
        let (n, k) = (gate.t.n, gate.t.k);
        let (m, mut dims) = rows_of(xs, k)?;
        let x: Vec<f32> = xs.flatten_all()?.to_vec1()?;
        let mut y = vec![0f32; m * n];
        let guard = gate.t.dev.lock()?;
        let ctx = guard.0;
        // SAFETY: x holds m * k floats, y m * n
        check(ctx, unsafe {
            turq_qmatmul_gate_up(ctx, gate.t.w, up.t.w, x.as_ptr().cast(), TURQ_ACT_F32, m as i64, k as i64, y.as_mut_ptr().cast(),
                                 TURQ_ACT_F32, n as i64, ptr::null(), ptr::null(), TURQ_ACTFN_SILU, TURQ_MEM_HOST)
        })?;
        if let Some(last) = dims.last_mut() {
            *last = n;
        }
        Tensor::from_vec(y, dims, xs.device())
    }

    /// `down_proj(act_fn(gate_proj(x)) * up_proj(x))`, the whole of `Qwen3MLP::forward` (src/models/qwen3.rs:161-167), SiLU.
    pub fn forward_mlp(gate: &HipQMatMul, up: &HipQMatMul, down: &HipQMatMul, xs: &Tensor) -> Result<Tensor> {
        let (k, n_out) = (gate.t.k, down.t.n);
        let (m, mut dims) = rows_of(xs, k)?;
        let x: Vec<f32> = xs.flatten_all()?.to_vec1()?;
        let mut y = vec![0f32; m * n_out];
        let guard = gate.t.dev.lock()?;
        let ctx = guard.0;
        // SAFETY: x holds m * k floats, y m * n_out
        check(ctx, unsafe {
            turq_mlp(ctx, gate.t.w, up.t.w, down.t.w, x.as_ptr().cast(), TURQ_ACT_F32, m as i64, k as i64, y.as_mut_ptr().cast(),
                     TURQ_ACT_F32, n_out as i64, ptr::null(), ptr::null(), ptr::null(), TURQ_ACTFN_SILU, TURQ_MEM_HOST)
        })?;
        if let Some(last) = dims.last_mut() {
            *last = n_out;
        }
        Tensor::from_vec(y, dims, xs.device())
    }
}

/// candle_nn's RmsNorm as `layers::norm::rms_norm` builds it from a GGUF file (src/models/layers/norm.rs:52-94).
#[derive(Clone)]
pub struct HipRmsNorm {
    dev: HipDevice,
    weight: Arc<Vec<f32>>,
    eps: f32,
}

impl HipRmsNorm {
    pub fn new(dev: &HipDevice, weight: &HipQTensor, eps: f64, is_gemma: bool) -> Result<Self> {
        let mut w: Vec<f32> = weight.dequantize(&Device::Cpu)?.flatten_all()?.to_vec1()?;
        if is_gemma {
            w.iter_mut().for_each(|v| *v += 1.0);
        }
        Ok(Self { dev: dev.clone(), weight: Arc::new(w), eps: eps as f32 })
    }
    /// `forward_multi(layers, self.forward(xs))` in one call: ln1 -> q / k / v (src/models/qwen3.rs:633-634, 272-274), the
    /// final norm -> lm_head; the norm is applied inside the matmul kernels where they can (turq_norm_qmatmul_multi)
    pub fn forward_then(&self, layers: &[&HipQMatMul], xs: &Tensor) -> Result<Vec<Tensor>> {
        let Some(first) = layers.first() else { return Ok(Vec::new()) };
        let k = first.t.k;
        let (m, dims) = rows_of(xs, k)?;
        if k != self.weight.len() || layers.iter().any(|l| l.t.k != k || l.dense) {
            let xn = self.forward(xs)?;
            return layers.iter().map(|l| l.forward(&xn)).collect();
        }
        let x: Vec<f32> = xs.flatten_all()?.to_vec1()?;
        let mut ys: Vec<Vec<f32>> = layers.iter().map(|l| vec![0f32; m * l.t.n]).collect();
        let ws: Vec<*const turq_weight> = layers.iter().map(|l| l.t.w as *const turq_weight).collect();
        let yp: Vec<*mut c_void> = ys.iter_mut().map(|y| y.as_mut_ptr().cast()).collect();
        let ld: Vec<i64> = layers.iter().map(|l| l.t.n as i64).collect();
        {
            let guard = self.dev.lock()?;
            let ctx = guard.0;
            // SAFETY: the arrays have one entry per layer and every buffer its full size; the norm weight holds k floats
            check(ctx, unsafe {
                turq_norm_qmatmul_multi(ctx, ws.len() as c_int, ws.as_ptr(), x.as_ptr().cast(), TURQ_ACT_F32, m as i64, k as i64,
                                        self.weight.as_ptr(), self.eps, yp.as_ptr(), TURQ_ACT_F32, ld.as_ptr(), ptr::null(), TURQ_MEM_HOST)
            })?;
        }
        ys.into_iter()
            .zip(layers)
            .map(|(y, l)| {
                let mut d = dims.clone();
                if let Some(last) = d.last_mut() {
                    *last = l.t.n;
                }
                Tensor::from_vec(y, d, xs.device())
            })
            .collect()
    }

    /// `xs + mlp(self.forward(xs))`, the second half of the decoder layer (src/models/qwen3.rs:637-640), in one call
    /// (turq_norm_mlp with TURQ_OUT_ACCUMULATE); the MLP's output width must be the input's
    pub fn forward_mlp_residual(&self, gate: &HipQMatMul, up: &HipQMatMul, down: &HipQMatMul, xs: &Tensor) -> Result<Tensor> {
        let (k, n_out) = (gate.t.k, down.t.n);
        let (m, dims) = rows_of(xs, k)?;
        if n_out != k || k != self.weight.len() {
            candle_core::bail!("shape mismatch: a residual MLP maps {} features to {}, the norm has {}", k, n_out, self.weight.len())
        }
        let x: Vec<f32> = xs.flatten_all()?.to_vec1()?;
        let mut y = x.clone();
        {
            let guard = self.dev.lock()?;
            let ctx = guard.0;
            // SAFETY: x and y hold m * k floats, the norm weight k
            check(ctx, unsafe {
                turq_norm_mlp(ctx, gate.t.w, up.t.w, down.t.w, x.as_ptr().cast(), TURQ_ACT_F32, m as i64, k as i64, self.weight.as_ptr(),
                              self.eps, y.as_mut_ptr().cast(), TURQ_ACT_F32 | TURQ_OUT_ACCUMULATE, n_out as i64, ptr::null(), ptr::null(),
                              ptr::null(), TURQ_ACTFN_SILU, TURQ_MEM_HOST)
            })?;
        }
        Tensor::from_vec(y, dims, xs.device())
    }

    pub fn forward(&self, xs: &Tensor) -> Result<Tensor> {
        let k = self.weight.len();
        let dims = xs.dims().to_vec();
        if dims.last() != Some(&k) {
            candle_core::bail!("shape mismatch in rms-norm: input {:?}, weight has {} elements", dims, k)
        }
        let x: Vec<f32> = xs.flatten_all()?.to_vec1()?;
        let m = if k == 0 { 0 } else { x.len() / k };
        let mut y = vec![0f32; x.len()];
        let guard = self.dev.lock()?;
        let ctx = guard.0;
        // SAFETY: x and y hold m * k floats, the weight k
        check(ctx, unsafe {
            turq_rms_norm(ctx, x.as_ptr().cast(), TURQ_ACT_F32, m as i64, k as i64, k as i64, self.weight.as_ptr(), self.eps,
                          y.as_mut_ptr().cast(), TURQ_ACT_F32, k as i64, TURQ_MEM_HOST)
        })?;
        Tensor::from_vec(y, dims, xs.device())
    }
}

struct Gguf(*mut turq_gguf);
// SAFETY: reads are serialised inside the library (one seek + read at a time)
unsafe impl Send for Gguf {}
unsafe impl Sync for Gguf {}
impl Drop for Gguf {
    fn drop(&mut self) {
        // SAFETY: the pointer came from turq_gguf_open and is closed once
        unsafe { turq_gguf_close(self.0) }
    }
}

/// The GGUF side of `QVarBuilder` (src/weights/gguf_varbuilder.rs) for tensors that go to the GPU.
#[derive(Clone)]
pub struct HipQVarBuilder {
    dev: HipDevice,
    gguf: Arc<Gguf>,
    path: Vec<String>,
}

impl HipQVarBuilder {
    pub fn from_gguf<P: AsRef<std::path::Path>>(p: P, dev: &HipDevice) -> Result<Self> {
        let c = CString::new(p.as_ref().to_string_lossy().as_bytes()).map_err(|e| Error::Msg(e.to_string()))?;
        let mut g = ptr::null_mut();
        // SAFETY: `c` is NUL-terminated, `g` a valid out pointer
        check(ptr::null(), unsafe { turq_gguf_open(c.as_ptr(), &mut g) })?;
        Ok(Self { dev: dev.clone(), gguf: Arc::new(Gguf(g)), path: Vec::new() })
    }
    pub fn pp<S: ToString>(&self, s: S) -> Self {
        let mut path = self.path.clone();
        path.push(s.to_string());
        Self { dev: self.dev.clone(), gguf: self.gguf.clone(), path }
    }
    fn full(&self, name: &str) -> String {
        if self.path.is_empty() {
            name.to_string()
        } else {
            format!("{}.{}", self.path.join("."), name)
        }
    }
    pub fn device(&self) -> &HipDevice {
        &self.dev
    }
    pub fn contains_key(&self, key: &str) -> bool {
        let Ok(c) = CString::new(self.full(key)) else { return false };
        // SAFETY: every out pointer may be null
        unsafe {
            turq_gguf_tensor_info(self.gguf.0, c.as_ptr(), ptr::null_mut(), ptr::null_mut(), ptr::null_mut(), ptr::null_mut(), ptr::null_mut())
                == TURQ_OK
        }
    }
    /// `get(shape, name)`: (n, k) for a matrix, (k,) for a vector; a mismatch is "shape mismatch for NAME, got .., expected .."
    pub fn get(&self, shape: &[usize], name: &str) -> Result<HipQTensor> {
        let (n, k, one_dim) = match *shape {
            [k] => (1i64, k as i64, true),
            [n, k] => (n as i64, k as i64, false),
            _ => candle_core::bail!("shape mismatch for {}: a linear weight has one or two dimensions, expected {:?}", name, shape),
        };
        self.load(name, n, k, one_dim)
    }
    pub fn get_no_shape(&self, name: &str) -> Result<HipQTensor> {
        self.load(name, -1, -1, false)
    }
    fn load(&self, name: &str, n: i64, k: i64, one_dim: bool) -> Result<HipQTensor> {
        let c = CString::new(self.full(name)).map_err(|e| Error::Msg(e.to_string()))?;
        let mut dt = 0 as c_int;
        // SAFETY: unused out pointers are null
        check(ptr::null(), unsafe {
            turq_gguf_tensor_info(self.gguf.0, c.as_ptr(), &mut dt, ptr::null_mut(), ptr::null_mut(), ptr::null_mut(), ptr::null_mut())
        })?;
        let quant = matches!(dt, TURQ_Q8_0 | TURQ_Q4_K | TURQ_Q5_K | TURQ_Q6_K);
        // matrices the matmul kernels read go to the tiled layout; vectors and dense tensors stay in GGUF order
        let layout = if quant && !one_dim { TURQ_LAYOUT_TILED } else { TURQ_LAYOUT_NATIVE };
        let mut w = ptr::null_mut();
        {
            let guard = self.dev.lock()?;
            // SAFETY: `w` is a valid out pointer
            check(guard.0, unsafe { turq_gguf_load_weight(guard.0, self.gguf.0, c.as_ptr(), n, k, layout, &mut w) })?;
        }
        HipQTensor::from_handle(&self.dev, w, one_dim)
    }
}

// ---- the patch against src/models/layers/linear.rs (lines 8-31 and 50-70) -------------------------------------------------
//
//  pub enum LinearX {
//      Standard(Linear),
//      Quantized { qmatmul: QMatMul, bias: Option<Tensor> },
// +    /// GGUF weights on an MI355X through libturq
// +    Hip { qmatmul: tur_hip::HipQMatMul, bias: Option<Tensor> },
//  }
//
//  impl Module for LinearX {
//      fn forward(&self, x: &Tensor) -> Result<Tensor> {
//          match self {
//              Self::Standard(linear) => linear.forward(x),
//              Self::Quantized { qmatmul, bias } => { ... }
// +            Self::Hip { qmatmul, bias } => {
// +                let out = qmatmul.forward(x)?;
// +                match bias {
// +                    Some(b) => out.broadcast_add(b),
// +                    None => Ok(out),
// +                }
// +            }
//          }
//      }
//  }
//
//  pub fn linear(in_dim: usize, out_dim: usize, vb: VarBuilderX) -> Result<LinearX> {
//      match &vb.0 {
//          Either::Left(inner_vb) => { ... }
// +        Either::Right(inner_vb) if inner_vb.hip().is_some() => {
// +            // the builder was opened on a HIP device: `hip()` is the HipQVarBuilder it keeps next to candle's Content
// +            let hvb = inner_vb.hip().ok_or_else(|| candle_core::Error::Msg("no HIP builder".into()))?;
// +            let qweight = hvb.get(&[out_dim, in_dim], "weight")?;
// +            let bias = hvb.get(&[out_dim], "bias").ok().map(|q| q.dequantize(&Device::Cpu)).transpose()?;
// +            Ok(LinearX::Hip { qmatmul: tur_hip::HipQMatMul::from_arc(qweight)?, bias })
// +        }
//          Either::Right(inner_vb) => { ... }
//      }
//  }
