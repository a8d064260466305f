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

/// The library's code of a floating element type (`mi_moe_dtype`).
fn float_code(a: &Array, what: &str) -> Result<i32, Exception> {
    match a.dtype() {
        Dtype::Bfloat16 => Ok(sys::MI_MOE_DTYPE_BF16),
        Dtype::Float16 => Ok(sys::MI_MOE_DTYPE_F16),
        Dtype::Float32 => Ok(sys::MI_MOE_DTYPE_F32),
        other => Err(Exception::custom(format!("[mi_moe] {what} must be bfloat16, float16 or float32, got {other:?}"))),
    }
}

/// An uninitialised array of `shape` in the element type of `like` (a floating type).
fn empty_like_dtype(like: &Array, shape: &[i32]) -> Result<Array, Exception> {
    let a = match like.dtype() {
        Dtype::Float32 => Array::zeros::<f32>(shape)?,
        Dtype::Float16 => Array::zeros::<half::f16>(shape)?,
        _ => Array::zeros::<half::bf16>(shape)?,
    };
    a.eval()?;
    Ok(a)
}

pub mod ops {
    use super::*;

    /// `(w_q, scales, biases)` of a `[rows, cols]` float32 matrix: `mi_moe_quantize_typed`.  Scales
    /// and biases come out in float32, the type of the input, as `ops::quantize` gives them
    /// (`mlx-rs/src/ops/quantization.rs:50-83`); cast them for a bfloat16 model.
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
        let mut s = Array::zeros::<f32>(&[rows as i32, (cols / group_size as i64) as i32])?;
        let mut b = Array::zeros::<f32>(&[rows as i32, (cols / group_size as i64) as i32])?;
        q.eval()?;
        s.eval()?;
        b.eval()?;
        check(unsafe {
            sys::mi_moe_quantize_typed(D::device_ptr(w) as *const f32, rows, cols, group_size, bits, sys::MI_MOE_DTYPE_F32, D::device_ptr_mut(&mut q) as *mut u32, D::device_ptr_mut(&mut s), D::device_ptr_mut(&mut b), D::hip_stream(stream))
        })?;
        Ok((q, s, b))
    }

    /// The quantisation mode of the reference's ops (`DEFAULT_MODE`, what `mlx-rs/src/ops/quantization.rs:213-227`
    /// hands to `mlx_gather_qmm` / `mlx_quantized_matmul` / `mlx_quantize`).  This library implements this mode only.
    pub const DEFAULT_MODE: &str = "affine";

    /// Refuses every mode but `"affine"`, in the shape of an MLX error.  The `*_with_mode` functions below
    /// stand where a caller of the `-sys` level passes a mode string.
    pub fn check_mode(mode: impl Into<Option<&'static str>>, op: &str) -> Result<(), Exception> {
        match mode.into().unwrap_or(DEFAULT_MODE) {
            "affine" => Ok(()),
            other => Err(Exception::custom(format!(
                "[{op}] Invalid quantization mode '{other}': mi_moe implements the 'affine' mode only (one scale and one bias per group)"
            ))),
        }
    }

    /// `gather_qmm` with the `mode` argument of `mlx_gather_qmm`; anything but `"affine"` is an error.
    #[allow(clippy::too_many_arguments)]
    pub fn gather_qmm_with_mode<'l, 'r, D: DeviceAccess>(
        x: &Array,
        w: &Array,
        scales: &Array,
        biases: &Array,
        lhs_indices: impl Into<Option<&'l Array>>,
        rhs_indices: impl Into<Option<&'r Array>>,
        transpose: impl Into<Option<bool>>,
        group_size: impl Into<Option<i32>>,
        bits: impl Into<Option<i32>>,
        mode: impl Into<Option<&'static str>>,
        sorted_indices: impl Into<Option<bool>>,
        stream: &Stream,
    ) -> Result<Array, Exception> {
        check_mode(mode, "gather_qmm")?;
        gather_qmm::<D>(x, w, scales, biases, lhs_indices, rhs_indices, transpose, group_size, bits, sorted_indices, stream)
    }

    /// `quantized_matmul` with the `mode` argument of `mlx_quantized_matmul`; anything but `"affine"` is an error.
    #[allow(clippy::too_many_arguments)]
    pub fn quantized_matmul_with_mode<D: DeviceAccess>(
        x: &Array,
        w: &Array,
        scales: &Array,
        biases: &Array,
        transpose: impl Into<Option<bool>>,
        group_size: impl Into<Option<i32>>,
        bits: impl Into<Option<i32>>,
        mode: impl Into<Option<&'static str>>,
        stream: &Stream,
    ) -> Result<Array, Exception> {
        check_mode(mode, "quantized_matmul")?;
        quantized_matmul::<D>(x, w, scales, biases, transpose, group_size, bits, stream)
    }

    /// `QuantizedLinear::forward` (`mlx-rs/src/nn/quantized.rs:363-386`): `quantized_matmul(x, w, scales, biases,
    /// true, ..)`, then `+ bias` when the layer has one (`mi_moe_quantized_linear_typed`).
    #[allow(clippy::too_many_arguments)]
    pub fn quantized_linear<'b, D: DeviceAccess>(
        x: &Array,
        w: &Array,
        scales: &Array,
        biases: &Array,
        linear_bias: impl Into<Option<&'b Array>>,
        group_size: impl Into<Option<i32>>,
        bits: impl Into<Option<i32>>,
        stream: &Stream,
    ) -> Result<Array, Exception> {
        let group_size = group_size.into().unwrap_or(DEFAULT_GROUP_SIZE);
        let bits = bits.into().unwrap_or(DEFAULT_BITS);
        let dt = float_code(x, "x")?;
        expect_dtype(w, Dtype::Uint32, "w")?;
        expect_dtype(scales, x.dtype(), "scales")?;
        expect_dtype(biases, x.dtype(), "biases")?;
        let linear_bias = linear_bias.into();
        let (k, n) = (x.dim(-1), w.dim(-2));
        if let Some(b) = linear_bias {
            expect_dtype(b, x.dtype(), "bias")?;
            if b.size() as i32 != n {
                return Err(Exception::custom("[mi_moe] quantized_linear: the bias must have one element per output column"));
            }
        }
        let m: i64 = x.shape()[..x.ndim() - 1].iter().map(|&d| d as i64).product();
        let mut ws_bytes = 0usize;
        check(unsafe { sys::mi_moe_quantized_matmul_workspace_size(m, k, bits, &mut ws_bytes) })?;
        let mut ws = D::device_buffer(ws_bytes.max(256))?;
        let mut shape = x.shape().to_vec();
        *shape.last_mut().unwrap() = n;
        let mut y = empty_like_dtype(x, &shape)?;
        check(unsafe {
            sys::mi_moe_quantized_linear_typed(D::device_ptr(x), D::device_ptr(w) as *const u32, D::device_ptr(scales), D::device_ptr(biases), linear_bias.map_or(std::ptr::null(), |b| D::device_ptr(b)), m, n, k, group_size, bits, dt, D::device_ptr_mut(&mut y), D::device_ptr_mut(&mut ws), ws_bytes, D::hip_stream(stream))
        })?;
        Ok(y)
    }

    /// `ops::dequantize` as the reference returns it (`mlx-rs/src/ops/quantization.rs:124-158`): the result has
    /// the element type of `scales` (`mi_moe_dequantize_native`).
    pub fn dequantize_native<D: DeviceAccess>(
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
        let dt = float_code(scales, "scales")?;
        expect_dtype(biases, scales.dtype(), "biases")?;
        let rows = w.dim(-2) as i64;
        let cols = w.dim(-1) as i64 * 32 / bits as i64;
        let mut out = empty_like_dtype(scales, &[rows as i32, cols as i32])?;
        check(unsafe {
            sys::mi_moe_dequantize_native(D::device_ptr(w) as *const u32, D::device_ptr(scales), D::device_ptr(biases), rows, cols, group_size, bits, dt, D::device_ptr_mut(&mut out), D::hip_stream(stream))
        })?;
        Ok(out)
    }

    /// `mi_moe_dequantize_typed`: float32 `[rows, cols]`; scales and biases in any floating type.
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
        let dt = float_code(scales, "scales")?;
        expect_dtype(biases, scales.dtype(), "biases")?;
        let rows = w.dim(-2) as i64;
        let cols = w.dim(-1) as i64 * 32 / bits as i64;
        let mut out = Array::zeros::<f32>(&[rows as i32, cols as i32])?;
        out.eval()?;
        check(unsafe {
            sys::mi_moe_dequantize_typed(D::device_ptr(w) as *const u32, D::device_ptr(scales), D::device_ptr(biases), rows, cols, group_size, bits, dt, D::device_ptr_mut(&mut out) as *mut f32, D::hip_stream(stream))
        })?;
        Ok(out)
    }

    /// `x [..., K]` times one quantized matrix, in any floating type (scales and biases in the type
    /// of `x`); `transpose` defaults to `false` as in `quantized_matmul`
    /// (`mlx-rs/src/ops/quantization.rs:91-122`).
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
        let transpose = transpose.into().unwrap_or(false);
        let group_size = group_size.into().unwrap_or(DEFAULT_GROUP_SIZE);
        let bits = bits.into().unwrap_or(DEFAULT_BITS);
        let dt = float_code(x, "x")?;
        expect_dtype(w, Dtype::Uint32, "w")?;
        expect_dtype(scales, x.dtype(), "scales")?;
        expect_dtype(biases, x.dtype(), "biases")?;
        let k = x.dim(-1);
        let m: i64 = x.shape()[..x.ndim() - 1].iter().map(|&d| d as i64).product();
        let n = if transpose { w.dim(-2) } else { w.dim(-1) * 32 / bits };
        let mut ws_bytes = 0usize;
        check(unsafe { sys::mi_moe_quantized_matmul_workspace_size(m, k, bits, &mut ws_bytes) })?;
        let mut ws = D::device_buffer(ws_bytes.max(256))?;
        let mut shape = x.shape().to_vec();
        *shape.last_mut().unwrap() = n;
        let mut y = empty_like_dtype(x, &shape)?;
        check(unsafe {
            sys::mi_moe_quantized_matmul_typed(D::device_ptr(x), D::device_ptr(w) as *const u32, D::device_ptr(scales), D::device_ptr(biases), m, n, k, transpose as i32, group_size, bits, dt, D::device_ptr_mut(&mut y), D::device_ptr_mut(&mut ws), ws_bytes, D::hip_stream(stream))
        })?;
        Ok(y)
    }

    /// `gather_qmm` with the argument list and the batch semantics of
    /// `mlx-rs/src/ops/quantization.rs:160-230`: `x` is `[..., M, K]` in any floating type, `w`
    /// `[..., N, K*bits/32]`; the index arrays (any shapes) address the flattened leading axes and
    /// are broadcast against each other; an absent one counts through its batch.  Returns
    /// `[*broadcast shape, M, N]`.
    #[allow(clippy::too_many_arguments)]
    pub fn gather_qmm<'l, 'r, D: DeviceAccess>(
        x: &Array,
        w: &Array,
        scales: &Array,
        biases: &Array,
        lhs_indices: impl Into<Option<&'l Array>>,
        rhs_indices: impl Into<Option<&'r Array>>,
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
        let dt = float_code(x, "x")?;
        expect_dtype(w, Dtype::Uint32, "w")?;
        expect_dtype(scales, x.dtype(), "scales")?;
        expect_dtype(biases, x.dtype(), "biases")?;
        if x.ndim() < 2 || w.ndim() < 2 {
            return Err(Exception::custom("[mi_moe] gather_qmm takes x [..., M, K] and w [..., N, K*bits/32]"));
        }
        let (m, k) = (x.dim(-2), x.dim(-1));
        let x_batch_shape = &x.shape()[..x.ndim() - 2];
        let w_batch_shape = &w.shape()[..w.ndim() - 2];
        let x_batch: i64 = x_batch_shape.iter().map(|&d| d as i64).product();
        let e: i64 = w_batch_shape.iter().map(|&d| d as i64).product();
        let n = if transpose { w.dim(-2) } else { w.dim(-1) * 32 / bits };
        // an absent index array counts through its batch, in the batch's shape
        let counted = |count: i64, shape: &[i32]| -> Result<Array, Exception> {
            Array::arange::<_, u32>(None, count, None)?.reshape(shape)
        };
        let lhs = match lhs_indices.into() {
            Some(a) => a.as_dtype(Dtype::Uint32)?,
            None => counted(x_batch, x_batch_shape)?,
        };
        let rhs = match rhs_indices.into() {
            Some(a) => a.as_dtype(Dtype::Uint32)?,
            None => counted(e, w_batch_shape)?,
        };
        let both = mlx_rs::ops::broadcast_arrays(&[&lhs, &rhs])?;
        let batch_shape = both[0].shape().to_vec();
        let lhs = both[0].flatten(None, None)?;
        let rhs = both[1].flatten(None, None)?;
        lhs.eval()?; // (materialised, row-major contiguous)
        rhs.eval()?;
        let n_idx = rhs.size() as i64;
        let mut ws_bytes = 0usize;
        check(unsafe { sys::mi_moe_gather_qmm_workspace_size(e.clamp(1, 512) as i32, n_idx, m, &mut ws_bytes) })?;
        let mut ws = D::device_buffer(ws_bytes.max(256))?;
        let mut shape = batch_shape;
        shape.push(m);
        shape.push(n);
        let mut y = empty_like_dtype(x, &shape)?;
        check(unsafe {
            sys::mi_moe_gather_qmm_typed(D::device_ptr(x), D::device_ptr(w) as *const u32, D::device_ptr(scales), D::device_ptr(biases), D::device_ptr(&lhs) as *const u32, D::device_ptr(&rhs) as *const u32, n_idx, x_batch, m, n, k, e as i32, transpose as i32, group_size, bits, sorted as i32, dt, D::device_ptr_mut(&mut y), D::device_ptr_mut(&mut ws), ws_bytes, D::hip_stream(stream))
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
    use mlx_rs::macros::{ModuleParameters, Quantizable};
    use mlx_rs::module::ModuleParameters as _; // freeze_parameters
    use mlx_rs::nn::Linear;
    use mlx_rs::quantization::{MaybeQuantized, Quantizable};
    use std::marker::PhantomData;

    /// One bank of E dense matrices `[E, N, K]`: what a switch layer holds before quantisation
    /// (the role `Linear` has for `QuantizedLinear`, `mlx-rs/src/nn/linear.rs:60-110`).
    /// This library has no dense expert product; the type exists so that the block can be built
    /// dense and quantised in process (`nn::quantize(model, None, None)`,
    /// `mlx-rs/src/nn/quantized.rs:25-36`, `examples/mistral/src/main.rs:186-193`).
    #[derive(Debug, Clone, ModuleParameters)]
    pub struct SwitchLinear {
        #[param]
        pub weight: Param<Array>, // [E, N, K]
    }

    /// One bank of E quantized matrices: the parameters of `QuantizedLinear`
    /// (`mlx-rs/src/nn/quantized.rs:254-279`) with a leading expert axis.  The packed weight is a
    /// parameter of this struct itself, so the flattened keys are the ones `mlx_lm.convert`
    /// writes (`...switch_mlp.gate_proj.{weight,scales,biases}`); `QuantizedLinear` nests it as
    /// `inner.weight` (`nn/quantized.rs:325-327`).
    #[derive(Debug, Clone, ModuleParameters)]
    pub struct QuantizedSwitchLinear {
        pub group_size: i32,
        pub bits: i32,

        #[param]
        pub weight: Param<Array>, // u32 [E, N, K*bits/32]

        #[param]
        pub scales: Param<Array>, // bf16 [E, N, K/group_size]

        #[param]
        pub biases: Param<Array>, // bf16 [E, N, K/group_size]
    }

    impl QuantizedSwitchLinear {
        /// Containers of the right shapes for a checkpoint to be loaded into
        /// (`load_safetensors` only overwrites parameters that exist, `module/module.rs:260-283`).
        pub fn zeros(n_experts: i32, n: i32, k: i32, group_size: i32, bits: i32) -> Result<Self, Exception> {
            let mut q = Self {
                group_size,
                bits,
                weight: Param::new(Array::zeros::<u32>(&[n_experts, n, k * bits / 32])?),
                scales: Param::new(Array::zeros::<half::bf16>(&[n_experts, n, k / group_size])?),
                biases: Param::new(Array::zeros::<half::bf16>(&[n_experts, n, k / group_size])?),
            };
            q.freeze_parameters(true); // as QuantizedLinear, nn/quantized.rs:275-276
            Ok(q)
        }
    }

    impl Quantizable for SwitchLinear {
        type Quantized = QuantizedSwitchLinear;
        type QuantizationError = Exception;

        /// Every row of every expert is quantised on its own, so the bank goes through
        /// `ops::quantize` (`mlx-rs/src/ops/quantization.rs:50-83`) as it is.
        fn try_into_quantized(self, group_size: i32, bits: i32) -> Result<QuantizedSwitchLinear, Exception> {
            let w = self.weight.value.as_dtype(Dtype::Bfloat16)?;
            let (wq, scales, biases) = mlx_rs::ops::quantize(&w, group_size, bits)?;
            let mut q = QuantizedSwitchLinear { group_size, bits, weight: Param::new(wq), scales: Param::new(scales), biases: Param::new(biases) };
            q.freeze_parameters(true);
            Ok(q)
        }
    }

    /// The three expert banks of a SwiGLU switch layer, with mlx-lm's field names.
    #[derive(Debug, Clone, ModuleParameters, Quantizable)]
    pub struct SwitchGlu {
        #[quantizable]
        #[param]
        pub gate_proj: MaybeQuantized<SwitchLinear>,

        #[quantizable]
        #[param]
        pub up_proj: MaybeQuantized<SwitchLinear>,

        #[quantizable]
        #[param]
        pub down_proj: MaybeQuantized<SwitchLinear>,
    }

    /// The library handle and what it was created from.  Kept apart from the block so that the
    /// block itself has no `Drop` (the derived `Quantizable` moves the fields out of `self`,
    /// `mlx-macros/src/quantizable.rs:76-88`).
    #[derive(Debug)]
    struct Bound {
        handle: sys::mi_moe_handle,
        pointers: [usize; 11], // device addresses of the ten weight arrays and the router bias
        config: [i32; 7],
    }

    impl Drop for Bound {
        fn drop(&mut self) {
            if !self.handle.is_null() {
                unsafe { sys::mi_moe_destroy(self.handle) };
            }
        }
    }

    /// Router + experts where the dense `Mlp` stands in a decoder layer
    /// (`mlx-lm/src/models/qwen3.rs:204-255`, field `mlp` of `TransformerBlock`, `:257-275`):
    /// the flattened parameter keys below `mlp.` are `gate.weight` (and `gate.bias` when the
    /// router has one) and `switch_mlp.{gate_proj,up_proj,down_proj}.{weight,scales,biases}`.
    /// `forward` is one library call.
    #[derive(Debug, ModuleParameters, Quantizable)]
    pub struct SparseMoeBlock<D: DeviceAccess> {
        /// bias-free `Linear` `[E, H]` in bf16, never quantised (`mlx-rs/src/nn/linear.rs:84-96`);
        /// a bias, if present, is added to the logits before they are rounded to bf16
        #[param]
        pub gate: Linear,

        #[quantizable]
        #[param]
        pub switch_mlp: SwitchGlu,

        pub top_k: i32,
        pub norm_topk_prob: bool,
        pub softmax_after_topk: bool, // Mixtral
        pub stream: Stream,

        bound: Option<Bound>,
        router_bias_f32: Option<Array>, // gate.bias as float32, the form the library takes
        workspace: Option<Array>,
        workspace_tokens: i64,
        _d: PhantomData<D>,
    }

    impl<D: DeviceAccess> SparseMoeBlock<D> {
        pub fn new(gate: Linear, switch_mlp: SwitchGlu, top_k: i32, norm_topk_prob: bool, softmax_after_topk: bool, stream: Stream) -> Self {
            Self { gate, switch_mlp, top_k, norm_topk_prob, softmax_after_topk, stream, bound: None, router_bias_f32: None, workspace: None, workspace_tokens: 0, _d: PhantomData }
        }

        /// A block with zero-filled quantized containers, ready for
        /// `load_safetensors` of a quantized checkpoint (`module/module.rs:260-283`).
        #[allow(clippy::too_many_arguments)]
        pub fn new_quantized(hidden: i32, n_experts: i32, intermediate: i32, top_k: i32, norm_topk_prob: bool, softmax_after_topk: bool, group_size: i32, bits: i32, stream: Stream) -> Result<Self, Exception> {
            let gate = Linear { weight: Param::new(Array::zeros::<half::bf16>(&[n_experts, hidden])?), bias: Param::new(None) };
            let bank = |n, k| QuantizedSwitchLinear::zeros(n_experts, n, k, group_size, bits).map(MaybeQuantized::Quantized);
            let switch_mlp = SwitchGlu { gate_proj: bank(intermediate, hidden)?, up_proj: bank(intermediate, hidden)?, down_proj: bank(hidden, intermediate)? };
            Ok(Self::new(gate, switch_mlp, top_k, norm_topk_prob, softmax_after_topk, stream))
        }

        fn quantized(m: &MaybeQuantized<SwitchLinear>, what: &str) -> Result<&QuantizedSwitchLinear, Exception> {
            match m {
                MaybeQuantized::Quantized(q) => Ok(q),
                MaybeQuantized::Original(_) => Err(Exception::custom(format!(
                    "[mi_moe] {what} is not quantized: this path runs MLX-affine 4/8-bit experts only; \
                     quantize the block (nn::quantize) or load a quantized checkpoint"
                ))),
            }
        }

        fn qmat(m: &QuantizedSwitchLinear) -> Result<sys::mi_moe_qmat, Exception> {
            expect_dtype(&m.weight, Dtype::Uint32, "weight")?;
            expect_dtype(&m.scales, Dtype::Bfloat16, "scales")?;
            expect_dtype(&m.biases, Dtype::Bfloat16, "biases")?;
            m.weight.eval()?;
            m.scales.eval()?;
            m.biases.eval()?;
            Ok(sys::mi_moe_qmat { w: D::device_ptr(&m.weight) as *const u32, scales: D::device_ptr(&m.scales) as *const u16, biases: D::device_ptr(&m.biases) as *const u16 })
        }

        /// Binds the weights and sizes the workspace for `t` tokens.  The handle keeps device
        /// addresses, so it is created again whenever a parameter has been replaced since
        /// (`load_safetensors`, `update`: `module/module.rs:70-80,260-283` assign new arrays).
        fn ensure(&mut self, t: i64) -> Result<(), Exception> {
            let (g, u, d) = (
                Self::quantized(&self.switch_mlp.gate_proj, "switch_mlp.gate_proj")?,
                Self::quantized(&self.switch_mlp.up_proj, "switch_mlp.up_proj")?,
                Self::quantized(&self.switch_mlp.down_proj, "switch_mlp.down_proj")?,
            );
            if g.bits != u.bits || g.bits != d.bits || g.group_size != u.group_size || g.group_size != d.group_size {
                return Err(Exception::custom("[mi_moe] the three expert banks must share bits and group_size"));
            }
            expect_dtype(&self.gate.weight, Dtype::Bfloat16, "gate.weight")?;
            self.gate.weight.eval()?;
            let score_mode = if self.softmax_after_topk {
                sys::MI_MOE_SCORE_TOPK_THEN_SOFTMAX
            } else if self.norm_topk_prob {
                sys::MI_MOE_SCORE_SOFTMAX_THEN_TOPK_RENORM
            } else {
                sys::MI_MOE_SCORE_SOFTMAX_THEN_TOPK
            };
            let cfg = sys::mi_moe_config {
                hidden: self.gate.weight.dim(1),
                n_experts: self.gate.weight.dim(0),
                top_k: self.top_k,
                intermediate: g.weight.dim(1),
                bits: g.bits,
                group_size: g.group_size,
                score_mode,
            };
            // the router's bias, once per distinct bias array, as float32
            let bias_src = self.gate.bias.value.as_ref().map(|b| D::device_ptr(b) as usize).unwrap_or(0);
            let bias_bound = self.bound.as_ref().map(|b| b.pointers[10]).unwrap_or(usize::MAX);
            if bias_src != bias_bound {
                self.router_bias_f32 = match self.gate.bias.value.as_ref() {
                    Some(b) => {
                        let f = b.as_dtype(Dtype::Float32)?;
                        f.eval()?;
                        Some(f)
                    }
                    None => None,
                };
            }
            let w = sys::mi_moe_weights {
                router_w: D::device_ptr(&self.gate.weight) as *const u16,
                router_bias: self.router_bias_f32.as_ref().map(|b| D::device_ptr(b) as *const f32).unwrap_or(std::ptr::null()),
                gate: Self::qmat(g)?,
                up: Self::qmat(u)?,
                down: Self::qmat(d)?,
            };
            let pointers = [
                w.router_w as usize, w.gate.w as usize, w.gate.scales as usize, w.gate.biases as usize,
                w.up.w as usize, w.up.scales as usize, w.up.biases as usize,
                w.down.w as usize, w.down.scales as usize, w.down.biases as usize, bias_src,
            ];
            let config = [cfg.hidden, cfg.n_experts, cfg.top_k, cfg.intermediate, cfg.bits, cfg.group_size, cfg.score_mode];
            let stale = match &self.bound {
                Some(b) => b.pointers != pointers || b.config != config,
                None => true,
            };
            if stale {
                self.bound = None; // destroys the old handle
                let mut handle: sys::mi_moe_handle = std::ptr::null_mut();
                check(unsafe { sys::mi_moe_create(&cfg, &w, &mut handle) })?;
                self.bound = Some(Bound { handle, pointers, config });
                self.workspace_tokens = 0; // the size depends on the configuration
            }
            if t > self.workspace_tokens || self.workspace.is_none() {
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
            expect_dtype(norm_weight, Dtype::Bfloat16, "norm_weight")?;
            h.eval()?;
            norm_weight.eval()?;
            let t = Self::tokens(h);
            self.ensure(t)?;
            let mut out = Array::zeros::<half::bf16>(h.shape())?;
            out.eval()?;
            let handle = self.bound.as_ref().unwrap().handle;
            let ws = self.workspace.as_mut().unwrap();
            let ws_bytes = ws.nbytes();
            check(unsafe {
                sys::mi_moe_forward_residual(handle, D::device_ptr(h) as *const u16, D::device_ptr(norm_weight) as *const u16, eps, t, D::device_ptr_mut(&mut out) as *mut u16, D::device_ptr_mut(ws), ws_bytes, std::ptr::null(), D::hip_stream(&self.stream))
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
            let handle = self.bound.as_ref().unwrap().handle;
            let ws = self.workspace.as_mut().unwrap();
            let ws_bytes = ws.nbytes();
            check(unsafe {
                sys::mi_moe_forward(handle, D::device_ptr(x) as *const u16, t, D::device_ptr_mut(&mut out) as *mut u16, D::device_ptr_mut(ws), ws_bytes, std::ptr::null(), D::hip_stream(&self.stream))
            })?;
            Ok(out)
        }

        /// Nothing in the block depends on the mode; the router is told, as `Mlp` tells its
        /// layers (`mlx-lm/src/models/qwen3.rs:249-254`).
        fn training_mode(&mut self, mode: bool) {
            self.gate.training_mode(mode);
        }
    }
}
