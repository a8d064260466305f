//! The quantized mixture-of-experts block of `libmi_moe.so` in mlx-rs's vocabulary.
//!
//! Shapes, defaults and error behaviour follow the functions this layer stands in for:
//! `ops::gather_qmm` / `quantized_matmul` / `quantize` / `dequantize`
//! (`mlx-rs/src/ops/quantization.rs:50-230`), `fast::rms_norm` (`mlx-rs/src/fast.rs:190-207`) and
//! a `Module<&Array>` (`mlx-rs/src/module/module.rs:28-50`) that sits where the dense `Mlp` sits
//! in a decoder layer (`mlx-lm/src/models/qwen3.rs:204-255,310-325`).
//!
//! Never compiled in the image this library is developed in (no rustc there).

use std::ffi::{c_void, CStr};
use std::os::raw::c_int;

use mi_moe_sys as sys;
use mlx_rs::error::Exception;
use mlx_rs::module::{Module, Param};
use mlx_rs::{Array, Dtype, Stream};

/// What this layer needs from an MLX build with a ROCm backend and mlx-rs does not expose today.
/// `Array::as_slice` (`mlx-rs/src/array/mod.rs:384-403`) is the host-memory counterpart.
pub trait DeviceAccess {
    /// Device address of an evaluated, row-major contiguous array (borrowed for its lifetime).
    fn device_ptr(a: &Array) -> *const c_void;
    fn device_ptr_mut(a: &mut Array) -> *mut c_void;
    /// The `hipStream_t` behind a stream; null = the default stream.
    fn hip_stream(s: &Stream) -> *mut c_void;
    /// Uninitialised device buffer of `bytes` bytes, 256-byte aligned, as a `Uint8` array.
    fn device_buffer(bytes: usize) -> Result<Array, Exception>;
}

/// Status -> `Exception`, the shape of `mlx-rs/src/utils/guard.rs:20-49` with the message pulled
/// from the library's thread-local slot instead of pushed through a handler.
fn check(status: c_int) -> Result<(), Exception> {
    if status == 0 {
        return Ok(());
    }
    let msg = unsafe { CStr::from_ptr(sys::mi_moe_last_error()) };
    Err(Exception::custom(msg.to_string_lossy().into_owned()))
}

fn expect_dtype(a: &Array, dt: Dtype, what: &str) -> Result<(), Exception> {
    if a.dtype() != dt {
        return Err(Exception::custom(format!("[mi_moe] {what} must be {dt:?}, got {:?}", a.dtype())));
    }
    Ok(())
}

pub const DEFAULT_GROUP_SIZE: i32 = 64; // mlx-rs/src/ops/quantization.rs:11-13
pub const DEFAULT_BITS: i32 = 4;

pub mod ops {
    use super::*;

    /// `(w_q, scales, biases)` of a `[rows, cols]` float32 matrix: `mi_moe_quantize`.
    pub fn quantize<D: DeviceAccess>(
        w: &Array,
        group_size: impl Into<Option<i32>>,
        bits: impl Into<Option<i32>>,
        stream: &Stream,
    ) -> Result<(Array, Array, Array), Exception> {
        let group_size = group_size.into().unwrap_or(DEFAULT_GROUP_SIZE);
        let bits = bits.into().unwrap_or(DEFAULT_BITS);
        expect_dtype(w, Dtype::Float32, "w")?;
        w.eval()?;
        let (rows, cols) = (w.dim(-2) as i64, w.dim(-1) as i64);
        let mut q = Array::zeros::<u32>(&[rows as i32, (cols * bits as i64 / 32) as i32])?;
        let mut s = Array::zeros::<half::bf16>(&[rows as i32, (cols / group_size as i64) as i32])?;
        let mut b = Array::zeros::<half::bf16>(&[rows as i32, (cols / group_size as i64) as i32])?;
        q.eval()?;
        s.eval()?;
        b.eval()?;
        check(unsafe {
            sys::mi_moe_quantize(D::device_ptr(w) as *const f32, rows, cols, group_size, bits, D::device_ptr_mut(&mut q) as *mut u32, D::device_ptr_mut(&mut s) as *mut u16, D::device_ptr_mut(&mut b) as *mut u16, D::hip_stream(stream))
        })?;
        Ok((q, s, b))
    }

    /// `mi_moe_dequantize`: float32 `[rows, cols]`.
    pub fn dequantize<D: DeviceAccess>(
        w: &Array,
        scales: &Array,
        biases: &Array,
        group_size: impl Into<Option<i32>>,
        bits: impl Into<Option<i32>>,
        stream: &Stream,
    ) -> Result<Array, Exception> {
        let group_size = group_size.into().unwrap_or(DEFAULT_GROUP_SIZE);
        let bits = bits.into().unwrap_or(DEFAULT_BITS);
        expect_dtype(w, Dtype::Uint32, "w")?;
        expect_dtype(scales, Dtype::Bfloat16, "scales")?;
        expect_dtype(biases, Dtype::Bfloat16, "biases")?;
        let rows = w.dim(-2) as i64;
        let cols = w.dim(-1) as i64 * 32 / bits as i64;
        let mut out = Array::zeros::<f32>(&[rows as i32, cols as i32])?;
        out.eval()?;
        check(unsafe {
            sys::mi_moe_dequantize(D::device_ptr(w) as *const u32, D::device_ptr(scales) as *const u16, D::device_ptr(biases) as *const u16, rows, cols, group_size, bits, D::device_ptr_mut(&mut out) as *mut f32, D::hip_stream(stream))
        })?;
        Ok(out)
    }

    /// `x [M, K]` times one quantized matrix; `transpose` defaults to `true` as in
    /// `quantized_matmul` (`mlx-rs/src/ops/quantization.rs:91-122`).
    #[allow(clippy::too_many_arguments)]
    pub fn quantized_matmul<D: DeviceAccess>(
        x: &Array,
        w: &Array,
        scales: &Array,
        biases: &Array,
        transpose: impl Into<Option<bool>>,
        group_size: impl Into<Option<i32>>,
        bits: impl Into<Option<i32>>,
        stream: &Stream,
    ) -> Result<Array, Exception> {
        let transpose = transpose.into().unwrap_or(true);
        let group_size = group_size.into().unwrap_or(DEFAULT_GROUP_SIZE);
        let bits = bits.into().unwrap_or(DEFAULT_BITS);
        expect_dtype(x, Dtype::Bfloat16, "x")?;
        expect_dtype(w, Dtype::Uint32, "w")?;
        let k = x.dim(-1);
        let m: i64 = x.shape()[..x.ndim() - 1].iter().map(|&d| d as i64).product();
        let n = if transpose { w.dim(-2) } else { w.dim(-1) * 32 / bits };
        let mut ws_bytes = 0usize;
        check(unsafe { sys::mi_moe_quantized_matmul_workspace_size(m, k, bits, &mut ws_bytes) })?;
        let mut ws = D::device_buffer(ws_bytes.max(256))?;
        let mut shape = x.shape().to_vec();
        *shape.last_mut().unwrap() = n;
        let mut y = Array::zeros::<half::bf16>(&shape)?;
        y.eval()?;
        check(unsafe {
            sys::mi_moe_quantized_matmul(D::device_ptr(x) as *const u16, D::device_ptr(w) as *const u32, D::device_ptr(scales) as *const u16, D::device_ptr(biases) as *const u16, m, n, k, transpose as i32, group_size, bits, D::device_ptr_mut(&mut y) as *mut u16, D::device_ptr_mut(&mut ws), ws_bytes, D::hip_stream(stream))
        })?;
        Ok(y)
    }

    /// `gather_qmm` with the argument list of `mlx-rs/src/ops/quantization.rs:180-230`.
    /// `x`: bf16 `[batch, M, K]`; `w`: `[E, N, K*bits/32]`; `rhs_indices` is required here
    /// (every switch layer passes it), `lhs_indices = None` pairs row `j` with index `j`.
    #[allow(clippy::too_many_arguments)]
    pub fn gather_qmm<'l, D: DeviceAccess>(
        x: &Array,
        w: &Array,
        scales: &Array,
        biases: &Array,
        lhs_indices: impl Into<Option<&'l Array>>,
        rhs_indices: &Array,
        transpose: impl Into<Option<bool>>,
        group_size: impl Into<Option<i32>>,
        bits: impl Into<Option<i32>>,
        sorted_indices: impl Into<Option<bool>>,
        stream: &Stream,
    ) -> Result<Array, Exception> {
        let transpose = transpose.into().unwrap_or(true);
        let group_size = group_size.into().unwrap_or(DEFAULT_GROUP_SIZE);
        let bits = bits.into().unwrap_or(DEFAULT_BITS);
        let sorted = sorted_indices.into().unwrap_or(false);
        let lhs = lhs_indices.into();
        expect_dtype(x, Dtype::Bfloat16, "x")?;
        expect_dtype(w, Dtype::Uint32, "w")?;
        expect_dtype(rhs_indices, Dtype::Uint32, "rhs_indices")?;
        if x.ndim() != 3 || w.ndim() != 3 {
            return Err(Exception::custom("[mi_moe] gather_qmm takes x [batch, M, K] and w [E, N, K*bits/32]"));
        }
        let (x_batch, m, k) = (x.dim(0) as i64, x.dim(1), x.dim(2));
        let e = w.dim(0);
        let n = if transpose { w.dim(1) } else { w.dim(2) * 32 / bits };
        let n_idx = rhs_indices.size() as i64;
        let mut ws_bytes = 0usize;
        check(unsafe { sys::mi_moe_gather_qmm_workspace_size(e, n_idx, m, &mut ws_bytes) })?;
        let mut ws = D::device_buffer(ws_bytes.max(256))?;
        let mut y = Array::zeros::<half::bf16>(&[n_idx as i32, m, n])?;
        y.eval()?;
        let lhs_ptr = lhs.map(|a| D::device_ptr(a) as *const u32).unwrap_or(std::ptr::null());
        check(unsafe {
            sys::mi_moe_gather_qmm(D::device_ptr(x) as *const u16, D::device_ptr(w) as *const u32, D::device_ptr(scales) as *const u16, D::device_ptr(biases) as *const u16, lhs_ptr, D::device_ptr(rhs_indices) as *const u32, n_idx, x_batch, m, n, k, e, transpose as i32, group_size, bits, sorted as i32, D::device_ptr_mut(&mut y) as *mut u16, D::device_ptr_mut(&mut ws), ws_bytes, D::hip_stream(stream))
        })?;
        Ok(y)
    }
}

pub mod fast {
    use super::*;

    /// `fast::rms_norm(x, weight, eps)` (`mlx-rs/src/fast.rs:190-207`) on bf16 rows.
    pub fn rms_norm<D: DeviceAccess>(x: &Array, weight: &Array, eps: f32, stream: &Stream) -> Result<Array, Exception> {
        expect_dtype(x, Dtype::Bfloat16, "x")?;
        expect_dtype(weight, Dtype::Bfloat16, "weight")?;
        let h = x.dim(-1);
        let t: i64 = x.shape()[..x.ndim() - 1].iter().map(|&d| d as i64).product();
        let mut out = Array::zeros::<half::bf16>(x.shape())?;
        out.eval()?;
        check(unsafe { sys::mi_moe_rms_norm(D::device_ptr(x) as *const u16, D::device_ptr(weight) as *const u16, eps, t, h, D::device_ptr_mut(&mut out) as *mut u16, D::hip_stream(stream)) })?;
        Ok(out)
    }
}

pub mod nn {
    use super::*;
    use std::marker::PhantomData;

    /// One bank of E quantized matrices: the fields of `QuantizedLinear`
    /// (`mlx-rs/src/nn/quantized.rs:254-279`) with a leading expert axis, named as
    /// `mlx_lm.convert` writes them (`…switch_mlp.gate_proj.{weight,scales,biases}`).
    #[derive(Debug, Clone)]
    pub struct QuantizedSwitchLinear {
        pub weight: Param<Array>, // u32 [E, N, K*bits/32]
        pub scales: Param<Array>, // bf16 [E, N, K/group_size]
        pub biases: Param<Array>, // bf16 [E, N, K/group_size]
    }

    #[derive(Debug, Clone)]
    pub struct SwitchGlu {
        pub gate_proj: QuantizedSwitchLinear,
        pub up_proj: QuantizedSwitchLinear,
        pub down_proj: QuantizedSwitchLinear,
    }

    /// Router + experts; `forward` is one library call.  In `mlx-lm` this struct additionally
    /// derives `ModuleParameters` with `#[param]` on `gate` and `switch_mlp` so that
    /// `load_safetensors` (`mlx-rs/src/module/module.rs:260-283`) finds
    /// `mlp.gate.weight` and `mlp.switch_mlp.*`.
    #[derive(Debug)]
    pub struct SparseMoeBlock<D: DeviceAccess> {
        pub gate: Param<Array>, // bf16 [E, H], bias-free Linear (mlx-rs/src/nn/linear.rs:84-96)
        pub switch_mlp: SwitchGlu,
        pub top_k: i32,
        pub norm_topk_prob: bool,
        pub softmax_after_topk: bool, // Mixtral
        pub bits: i32,
        pub group_size: i32,
        handle: sys::mi_moe_handle,
        workspace: Option<Array>,
        workspace_tokens: i64,
        stream: Stream,
        _d: PhantomData<D>,
    }

    impl<D: DeviceAccess> SparseMoeBlock<D> {
        #[allow(clippy::too_many_arguments)]
        pub fn new(gate: Array, switch_mlp: SwitchGlu, top_k: i32, norm_topk_prob: bool, softmax_after_topk: bool, bits: i32, group_size: i32, stream: Stream) -> Self {
            Self { gate: Param::new(gate), switch_mlp, top_k, norm_topk_prob, softmax_after_topk, bits, group_size, handle: std::ptr::null_mut(), workspace: None, workspace_tokens: 0, stream, _d: PhantomData }
        }

        fn config(&self) -> sys::mi_moe_config {
            let score_mode = if self.softmax_after_topk {
                sys::MI_MOE_SCORE_TOPK_THEN_SOFTMAX
            } else if self.norm_topk_prob {
                sys::MI_MOE_SCORE_SOFTMAX_THEN_TOPK_RENORM
            } else {
                sys::MI_MOE_SCORE_SOFTMAX_THEN_TOPK
            };
            sys::mi_moe_config {
                hidden: self.gate.dim(1),
                n_experts: self.gate.dim(0),
                top_k: self.top_k,
                intermediate: self.switch_mlp.gate_proj.weight.dim(1),
                bits: self.bits,
                group_size: self.group_size,
                score_mode,
            }
        }

        fn qmat(m: &QuantizedSwitchLinear) -> Result<sys::mi_moe_qmat, Exception> {
            m.weight.eval()?;
            m.scales.eval()?;
            m.biases.eval()?;
            Ok(sys::mi_moe_qmat { w: D::device_ptr(&m.weight) as *const u32, scales: D::device_ptr(&m.scales) as *const u16, biases: D::device_ptr(&m.biases) as *const u16 })
        }

        /// Binds the weights (once) and sizes the workspace for `t` tokens (when `t` grows).
        fn ensure(&mut self, t: i64) -> Result<(), Exception> {
            let cfg = self.config();
            if self.handle.is_null() {
                self.gate.eval()?;
                let w = sys::mi_moe_weights {
                    router_w: D::device_ptr(&self.gate) as *const u16,
                    router_bias: std::ptr::null(),
                    gate: Self::qmat(&self.switch_mlp.gate_proj)?,
                    up: Self::qmat(&self.switch_mlp.up_proj)?,
                    down: Self::qmat(&self.switch_mlp.down_proj)?,
                };
                check(unsafe { sys::mi_moe_create(&cfg, &w, &mut self.handle) })?;
            }
            if t > self.workspace_tokens {
                let mut bytes = 0usize;
                check(unsafe { sys::mi_moe_workspace_size(&cfg, t, &mut bytes) })?;
                self.workspace = Some(D::device_buffer(bytes)?);
                self.workspace_tokens = t;
            }
            Ok(())
        }

        fn tokens(x: &Array) -> i64 {
            x.shape()[..x.ndim() - 1].iter().map(|&d| d as i64).product()
        }

        /// `h + mlp(post_attention_layernorm(h))` of a decoder layer in one call
        /// (`mlx-lm/src/models/qwen3.rs:310-325`).
        pub fn forward_residual(&mut self, h: &Array, norm_weight: &Array, eps: f32) -> Result<Array, Exception> {
            expect_dtype(h, Dtype::Bfloat16, "h")?;
            h.eval()?;
            norm_weight.eval()?;
            let t = Self::tokens(h);
            self.ensure(t)?;
            let mut out = Array::zeros::<half::bf16>(h.shape())?;
            out.eval()?;
            let ws = self.workspace.as_mut().unwrap();
            let ws_bytes = ws.nbytes();
            check(unsafe {
                sys::mi_moe_forward_residual(self.handle, D::device_ptr(h) as *const u16, D::device_ptr(norm_weight) as *const u16, eps, t, D::device_ptr_mut(&mut out) as *mut u16, D::device_ptr_mut(ws), ws_bytes, std::ptr::null(), D::hip_stream(&self.stream))
            })?;
            Ok(out)
        }
    }

    impl<D: DeviceAccess + std::fmt::Debug> Module<&Array> for SparseMoeBlock<D> {
        type Output = Array;
        type Error = Exception;

        /// `[B, L, H] -> [B, L, H]`, bf16.
        fn forward(&mut self, x: &Array) -> Result<Array, Exception> {
            expect_dtype(x, Dtype::Bfloat16, "x")?;
            x.eval()?; // materialise, as Array::as_slice does before handing out a pointer
            let t = Self::tokens(x);
            self.ensure(t)?;
            let mut out = Array::zeros::<half::bf16>(x.shape())?;
            out.eval()?;
            let ws = self.workspace.as_mut().unwrap();
            let ws_bytes = ws.nbytes();
            check(unsafe {
                sys::mi_moe_forward(self.handle, D::device_ptr(x) as *const u16, t, D::device_ptr_mut(&mut out) as *mut u16, D::device_ptr_mut(ws), ws_bytes, std::ptr::null(), D::hip_stream(&self.stream))
            })?;
            Ok(out)
        }

        fn training_mode(&mut self, _mode: bool) {} // frozen weights, as QuantizedLinear (nn/quantized.rs:275-276)
    }

    impl<D: DeviceAccess> Drop for SparseMoeBlock<D> {
        fn drop(&mut self) {
            if !self.handle.is_null() {
                unsafe { sys::mi_moe_destroy(self.handle) };
            }
        }
    }
}
