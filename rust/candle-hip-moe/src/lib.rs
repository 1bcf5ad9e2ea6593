//! candle's quantized sparse-MoE block and quantized projections on an AMD MI355X (gfx950).
//!
//! `HipSparseMoe` stands in for the `MlpOrMoe::MoE` arm of
//! `candle-transformers/src/models/quantized_llama.rs:133-211`: same `forward(&Tensor) -> Result<Tensor>`,
//! exposed both as a `Module` and as a `CustomOp1` (`candle-core/src/custom_op.rs:7-41`).  `HipQMatMul` stands
//! in for the `QMatMul::QTensor` arm (`candle-core/src/quantized/mod.rs:428-447, 533-537`) and keeps the
//! reference's op name, "qmatmul" (`quantized/mod.rs:470-473`).  `HipRmsNorm` is `RmsNorm`
//! (`candle-transformers/src/quantized_nn.rs:100-126`).
//!
//! candle's `Device` has no HIP variant (`candle-core/src/device.rs:16-20`): tensors stay CPU tensors, the ops
//! receive host f32 storage in `cpu_fwd` and return host f32 storage; the quantized weights live on the GPU
//! inside the op object.  Errors of the library become `candle::Error::Msg` through `bail!`.
#![allow(clippy::missing_safety_doc)]

use candle::quantized::{GgmlDType, QTensor};
use candle::{bail, CpuStorage, CustomOp1, DType, Layout, Module, Result, Shape, Tensor};
use std::ffi::{CStr, CString};
use std::os::raw::{c_char, c_void};
use std::path::Path;

/// The C ABI of libcandle_amd_moe.so, as declared in include/candle_amd_moe.h.
pub mod ffi {
    use std::os::raw::{c_char, c_void};

    #[repr(C)]
    pub struct MoeLayer {
        _private: [u8; 0],
    }
    #[repr(C)]
    pub struct MoeQLinear {
        _private: [u8; 0],
    }
    #[repr(C)]
    pub struct MoeGguf {
        _private: [u8; 0],
    }

    #[repr(C)]
    pub struct MoeDesc {
        pub hidden: i64,
        pub ffn: i64,
        pub n_experts: i64,
        pub top_k: i64,
        pub ggml_dtype: i32,
        pub norm_topk: i32,
        pub gate: *const f32,
        pub gate_bias: *const f32,
        pub w1: *const *const c_void,
        pub w3: *const *const c_void,
        pub w2: *const *const c_void,
        pub shared_ffn: i64,
        pub shared_w1: *const c_void,
        pub shared_w3: *const c_void,
        pub shared_w2: *const c_void,
        pub shared_gate: *const f32,
        pub rms_alpha: *const f32,
        pub rms_eps: f32,
        pub ggml_dtype_down: i32,
        pub gate_dtype: i32,
        pub gate_blocks: *const c_void,
    }

    extern "C" {
        pub fn moe_layer_create(desc: *const MoeDesc, out: *mut *mut MoeLayer) -> i32;
        pub fn moe_layer_destroy(layer: *mut MoeLayer);
        pub fn moe_layer_shape(layer: *const MoeLayer, hidden: *mut i64, ffn: *mut i64, n_experts: *mut i64, top_k: *mut i64) -> i32;
        pub fn moe_layer_forward(layer: *mut MoeLayer, x: *const f32, n_tokens: i64, y: *mut f32) -> i32;
        pub fn moe_layer_forward_device(layer: *mut MoeLayer, d_x: *const c_void, n_tokens: i64, d_y: *mut c_void, hip_stream: *mut c_void) -> i32;
        pub fn moe_layer_forward_device_noalloc(layer: *mut MoeLayer, d_x: *const c_void, n_tokens: i64, d_y: *mut c_void, hip_stream: *mut c_void) -> i32;
        pub fn moe_static_scratch_bytes() -> i64;
        pub fn moe_stack_forward_device(layers: *const *mut MoeLayer, n_layers: i64, d_x: *const c_void, n_tokens: i64, d_y: *mut c_void, hip_stream: *mut c_void) -> i32;
        pub fn moe_qmatmul(ggml_dtype: i32, w_blocks: *const c_void, n: i64, k: i64, x: *const f32, m: i64, y: *mut f32) -> i32;
        pub fn moe_qlinear_create(ggml_dtype: i32, w_blocks: *const c_void, n: i64, k: i64, out: *mut *mut MoeQLinear) -> i32;
        pub fn moe_qlinear_destroy(q: *mut MoeQLinear);
        pub fn moe_qlinear_forward(q: *mut MoeQLinear, x: *const f32, m: i64, y: *mut f32) -> i32;
        pub fn moe_qlinear_forward_device(q: *mut MoeQLinear, d_x: *const c_void, m: i64, d_y: *mut c_void, hip_stream: *mut c_void) -> i32;
        pub fn moe_qlinear_dequantize(q: *mut MoeQLinear, out: *mut f32, n_elems: i64) -> i32;
        pub fn moe_qlinear_shape(q: *const MoeQLinear, n: *mut i64, k: *mut i64, ggml_dtype: *mut i32) -> i32;
        pub fn moe_rms_norm(x: *const f32, alpha: *const f32, eps: f32, rows: i64, hidden: i64, y: *mut f32) -> i32;
        pub fn moe_add_rms_norm_device(d_x: *const c_void, d_residual: *const c_void, d_alpha: *const c_void, eps: f32, rows: i64, hidden: i64, d_sum: *mut c_void, d_y: *mut c_void, hip_stream: *mut c_void) -> i32;
        pub fn moe_dequantize(ggml_dtype: i32, blocks: *const c_void, n_elems: i64, out: *mut f32) -> i32;
        pub fn moe_quantize_weights(ggml_dtype: i32, x: *const f32, n_elems: i64, out_blocks: *mut c_void) -> i32;
        pub fn moe_gguf_open(path: *const c_char, out: *mut *mut MoeGguf) -> i32;
        pub fn moe_gguf_close(file: *mut MoeGguf);
        pub fn moe_layer_create_from_gguf(file: *const MoeGguf, layer_index: i32, norm_topk: i32, out: *mut *mut MoeLayer) -> i32;
        pub fn moe_qlinear_create_from_gguf(file: *const MoeGguf, tensor_name: *const c_char, out: *mut *mut MoeQLinear) -> i32;
        pub fn moe_last_error() -> *const c_char;
        pub fn moe_device_arch() -> *const c_char;
    }
}

fn last_error() -> String {
    // SAFETY: the library returns a NUL-terminated string owned by the calling thread's state
    unsafe { CStr::from_ptr(ffi::moe_last_error()) }.to_string_lossy().into_owned()
}

fn check(rc: i32) -> Result<()> {
    if rc != 0 {
        bail!("{}", last_error())
    }
    Ok(())
}

/// GgmlDType -> the numbering of `GgmlDType::to_u32` (candle-core/src/quantized/mod.rs:176-196), which is also the
/// library's (`MOE_GGML_*`).
fn ggml_id(d: GgmlDType) -> Result<i32> {
    Ok(match d {
        GgmlDType::Q4_0 => 2,
        GgmlDType::Q4_1 => 3,
        GgmlDType::Q5_0 => 6,
        GgmlDType::Q5_1 => 7,
        GgmlDType::Q8_0 => 8,
        GgmlDType::Q2K => 10,
        GgmlDType::Q3K => 11,
        GgmlDType::Q4K => 12,
        GgmlDType::Q5K => 13,
        GgmlDType::Q6K => 14,
        other => bail!("candle-hip-moe: unsupported weight dtype {other:?}"),
    })
}

/// Name of the GPU the library runs on ("gfx950..."), or the reason it cannot run.
pub fn device_arch() -> Result<String> {
    let p = unsafe { ffi::moe_device_arch() };
    if p.is_null() {
        bail!("{}", last_error())
    }
    Ok(unsafe { CStr::from_ptr(p) }.to_string_lossy().into_owned())
}

/// The f32 rows behind a contiguous CPU f32 storage, as `QTensor`'s own `cpu_fwd` takes them
/// (candle-core/src/quantized/mod.rs:480-482, 501): anything else is an error, not a conversion.
fn contiguous_f32<'a>(storage: &'a CpuStorage, layout: &Layout, who: &str) -> Result<&'a [f32]> {
    if !layout.is_contiguous() {
        bail!("{who}: input tensor is not contiguous {layout:?}")
    }
    let slice = storage.as_slice::<f32>()?;
    let start = layout.start_offset();
    Ok(&slice[start..start + layout.shape().elem_count()])
}

fn f32_vec(t: &Tensor) -> Result<Vec<f32>> {
    t.to_dtype(DType::F32)?.flatten_all()?.to_vec1::<f32>()
}

// ------------------------------------------------------------------------------------------------ MoE block

/// One always-on shared expert behind a sigmoid gate (qwen2_moe.rs:315-319).
pub struct SharedExpert<'a> {
    pub w1: &'a QTensor,   // gate_proj  [shared_ffn, hidden]
    pub w2: &'a QTensor,   // down_proj  [hidden, shared_ffn]
    pub w3: &'a QTensor,   // up_proj    [shared_ffn, hidden]
    pub gate: &'a Tensor,  // shared_expert_gate [1, hidden] or [hidden]
}

/// Everything `MlpOrMoe::MoE` holds (quantized_llama.rs:133-141), plus the options of the other MoE flavours the
/// library covers.  `experts[e] = (w1, w2, w3)` in the order of `Mlp` (feed_forward_w1 / w2 / w3, :117-122).
pub struct HipSparseMoeConfig<'a> {
    pub gate: &'a Tensor,                         // ffn_gate_inp, dequantised: [n_experts, hidden]
    pub gate_quantized: Option<&'a QTensor>,      // the same tensor kept quantised (any dtype but F32 / F16 / BF16): its logits
                                                  // are then the quantised product the reference's QMatMul::QTensor arm computes
    pub experts: &'a [(QTensor, QTensor, QTensor)],
    pub n_expert_used: usize,                     // 0 is accepted: the reference then returns zeros (:167, :507-512)
    pub norm_topk: bool,                          // Mixtral: true (:175-178); qwen2-moe's norm_topk_prob
    pub gate_bias: Option<&'a Tensor>,            // [n_experts], added to the logits (none in the reference's models)
    pub shared: Option<SharedExpert<'a>>,
    pub rms_norm: Option<(&'a Tensor, f64)>,      // ffn_norm weight and eps: y = x + moe(rms_norm(x)) (:886-890)
}

/// The sparse-MoE block with its quantized experts resident on the GPU.
pub struct HipSparseMoe {
    handle: *mut ffi::MoeLayer,
    hidden: usize,
}
// QuantizedType is Send + Sync (candle-core/src/quantized/mod.rs:256); calls on one layer are serialised inside
// the library.
unsafe impl Send for HipSparseMoe {}
unsafe impl Sync for HipSparseMoe {}

impl HipSparseMoe {
    /// Mixtral flavour: renormalised top-k, no bias, no shared expert, no fused norm.
    pub fn new(gate: &Tensor, experts: &[(QTensor, QTensor, QTensor)], n_expert_used: usize) -> Result<Self> {
        Self::with_config(HipSparseMoeConfig {
            gate,
            gate_quantized: None,
            experts,
            n_expert_used,
            norm_topk: true,
            gate_bias: None,
            shared: None,
            rms_norm: None,
        })
    }

    pub fn with_config(cfg: HipSparseMoeConfig<'_>) -> Result<Self> {
        let (n_experts, hidden) = cfg.gate.dims2()?;
        if cfg.experts.len() != n_experts || n_experts == 0 {
            bail!("HipSparseMoe: the gate has {n_experts} rows for {} experts", cfg.experts.len())
        }
        let (ffn, h1) = cfg.experts[0].0.shape().dims2()?;
        if h1 != hidden {
            bail!("HipSparseMoe: w1 is {:?}, the gate has hidden size {hidden}", cfg.experts[0].0.shape())
        }
        let dtype = cfg.experts[0].0.dtype();
        let dtype_down = cfg.experts[0].1.dtype();
        for (e, (w1, w2, w3)) in cfg.experts.iter().enumerate() {
            if w1.shape().dims2()? != (ffn, hidden) || w3.shape().dims2()? != (ffn, hidden) || w2.shape().dims2()? != (hidden, ffn) {
                bail!("HipSparseMoe: expert {e} has shapes {:?} {:?} {:?}", w1.shape(), w2.shape(), w3.shape())
            }
            if w1.dtype() != dtype || w3.dtype() != dtype || w2.dtype() != dtype_down {
                bail!("HipSparseMoe: expert {e} differs in dtype from expert 0")
            }
        }
        let gate = f32_vec(cfg.gate)?;
        // `gate_quantized`: the router as the reference runs it when `ffn_gate_inp` is not F32 / F16 / BF16
        let gate_q = match cfg.gate_quantized {
            Some(q) => {
                if q.shape().dims2()? != (n_experts, hidden) {
                    bail!("HipSparseMoe: the quantised gate is {:?}, expected [{n_experts}, {hidden}]", q.shape())
                }
                Some((q.dtype(), q.data()?))
            }
            None => None,
        };
        let gate_bias = cfg.gate_bias.map(f32_vec).transpose()?;
        if let Some(b) = &gate_bias {
            if b.len() != n_experts {
                bail!("HipSparseMoe: gate_bias has {} elements for {n_experts} experts", b.len())
            }
        }
        // QTensor::data() returns Result<Cow<[u8]>> (quantized/mod.rs:394-396): the Cows are kept alive in `bytes`
        // until moe_layer_create has copied the blocks to the device
        let mut bytes = Vec::with_capacity(3 * n_experts);
        for (w1, w2, w3) in cfg.experts.iter() {
            bytes.push(w1.data()?);
            bytes.push(w2.data()?);
            bytes.push(w3.data()?);
        }
        let p1: Vec<*const c_void> = (0..n_experts).map(|e| bytes[3 * e].as_ptr() as *const c_void).collect();
        let p2: Vec<*const c_void> = (0..n_experts).map(|e| bytes[3 * e + 1].as_ptr() as *const c_void).collect();
        let p3: Vec<*const c_void> = (0..n_experts).map(|e| bytes[3 * e + 2].as_ptr() as *const c_void).collect();

        let null = std::ptr::null::<c_void>();
        let (mut shared_ffn, mut s1, mut s2, mut s3) = (0i64, null, null, null);
        let mut shared_gate = Vec::new();
        let shared_bytes;
        if let Some(s) = &cfg.shared {
            let (fs, hs) = s.w1.shape().dims2()?;
            if hs != hidden || s.w3.shape().dims2()? != (fs, hidden) || s.w2.shape().dims2()? != (hidden, fs) {
                bail!("HipSparseMoe: shared expert has shapes {:?} {:?} {:?}", s.w1.shape(), s.w2.shape(), s.w3.shape())
            }
            if s.w1.dtype() != dtype || s.w3.dtype() != dtype || s.w2.dtype() != dtype_down {
                bail!("HipSparseMoe: the shared expert differs in dtype from the routed experts")
            }
            shared_gate = f32_vec(s.gate)?;
            if shared_gate.len() != hidden {
                bail!("HipSparseMoe: shared_expert_gate has {} elements, hidden is {hidden}", shared_gate.len())
            }
            shared_bytes = (s.w1.data()?, s.w2.data()?, s.w3.data()?);
            shared_ffn = fs as i64;
            s1 = shared_bytes.0.as_ptr() as *const c_void;
            s2 = shared_bytes.1.as_ptr() as *const c_void;
            s3 = shared_bytes.2.as_ptr() as *const c_void;
        }
        let (alpha, eps) = match cfg.rms_norm {
            Some((w, eps)) => {
                let a = f32_vec(w)?;
                if a.len() != hidden {
                    bail!("HipSparseMoe: the norm weight has {} elements, hidden is {hidden}", a.len())
                }
                (a, eps as f32)
            }
            None => (Vec::new(), 0f32),
        };
        let id = ggml_id(dtype)?;
        let id_down = ggml_id(dtype_down)?;
        let desc = ffi::MoeDesc {
            hidden: hidden as i64,
            ffn: ffn as i64,
            n_experts: n_experts as i64,
            top_k: cfg.n_expert_used as i64,
            ggml_dtype: id,
            norm_topk: cfg.norm_topk as i32,
            gate: gate.as_ptr(),
            gate_bias: gate_bias.as_ref().map_or(std::ptr::null(), |b| b.as_ptr()),
            w1: p1.as_ptr(),
            w3: p3.as_ptr(),
            w2: p2.as_ptr(),
            shared_ffn,
            shared_w1: s1,
            shared_w3: s3,
            shared_w2: s2,
            shared_gate: if shared_gate.is_empty() { std::ptr::null() } else { shared_gate.as_ptr() },
            rms_alpha: if alpha.is_empty() { std::ptr::null() } else { alpha.as_ptr() },
            rms_eps: eps,
            // Q4_K_M files store ffn_down of some layers as Q6K beside Q4K gate / up matrices (0 = same dtype)
            ggml_dtype_down: if id_down == id { 0 } else { id_down },
            // a router tensor the reference keeps quantised (QMatMul::from_arc, quantized/mod.rs:428-447)
            gate_dtype: gate_q.as_ref().map_or(Ok(0), |(d, _)| ggml_id(*d))?,
            gate_blocks: gate_q.as_ref().map_or(null, |(_, b)| b.as_ptr() as *const c_void),
        };
        let mut handle = std::ptr::null_mut();
        // SAFETY: every pointer in desc refers to a live buffer of the size the header states; the library only
        // borrows them for the call
        check(unsafe { ffi::moe_layer_create(&desc, &mut handle) })?;
        Ok(Self { handle, hidden })
    }

    /// The MoE arm of `ModelWeights::from_gguf` for layer `layer_index` (quantized_llama.rs:506-512, 553-578), read
    /// straight from the file: `llama.expert_count`, `llama.expert_used_count`, `blk.{l}.ffn_gate_inp.weight`,
    /// `blk.{l}.ffn_{gate,down,up}.{i}.weight`.
    pub fn from_gguf<P: AsRef<Path>>(path: P, layer_index: usize) -> Result<Self> {
        let file = GgufFile::open(path)?;
        let mut handle = std::ptr::null_mut();
        check(unsafe { ffi::moe_layer_create_from_gguf(file.0, layer_index as i32, 1, &mut handle) })?;
        let mut this = Self { handle, hidden: 0 };   // dropped (and the layer destroyed) if the next call fails
        let mut hidden = 0i64;
        let null = std::ptr::null_mut();
        check(unsafe { ffi::moe_layer_shape(this.handle, &mut hidden, null, null, null) })?;
        this.hidden = hidden as usize;
        Ok(this)
    }

    /// The forward on device pointers (HIP memory the caller owns), enqueued on `hip_stream` (null = default
    /// stream) without synchronising: for hosts that keep activations on the GPU.  `no_alloc` selects the entry
    /// point that allocates nothing (workspace in the library's static device array, batches up to what it holds).
    pub unsafe fn forward_device(&self, d_x: *const c_void, n_tokens: usize, d_y: *mut c_void, hip_stream: *mut c_void, no_alloc: bool) -> Result<()> {
        let rc = if no_alloc {
            ffi::moe_layer_forward_device_noalloc(self.handle, d_x, n_tokens as i64, d_y, hip_stream)
        } else {
            ffi::moe_layer_forward_device(self.handle, d_x, n_tokens as i64, d_y, hip_stream)
        };
        check(rc)
    }
}

/// The MoE blocks of consecutive layers on device pointers (HIP memory the caller owns), enqueued on `hip_stream`
/// without synchronising: `y = layers[n-1](... layers[0](x))`, the same bits as the layers' own forwards one after
/// the other, with each layer's combine pass folded into the next layer's front kernel at decode batch sizes.
pub unsafe fn stack_forward_device(layers: &[&HipSparseMoe], d_x: *const c_void, n_tokens: usize, d_y: *mut c_void, hip_stream: *mut c_void) -> Result<()> {
    let handles: Vec<*mut ffi::MoeLayer> = layers.iter().map(|l| l.handle).collect();
    check(ffi::moe_stack_forward_device(handles.as_ptr(), handles.len() as i64, d_x, n_tokens as i64, d_y, hip_stream))
}

impl CustomOp1 for HipSparseMoe {
    fn name(&self) -> &'static str {
        "hip-sparse-moe"
    }

    fn cpu_fwd(&self, storage: &CpuStorage, layout: &Layout) -> Result<(CpuStorage, Shape)> {
        let xs = contiguous_f32(storage, layout, "hip-sparse-moe")?;
        let dims = layout.shape().dims();
        if dims.last().copied() != Some(self.hidden) {
            bail!("hip-sparse-moe: input {:?} does not end in the hidden size {}", layout.shape(), self.hidden)
        }
        let n_tokens = xs.len() / self.hidden;
        let mut ys = vec![0f32; xs.len()];
        // SAFETY: xs and ys hold n_tokens * hidden floats
        check(unsafe { ffi::moe_layer_forward(self.handle, xs.as_ptr(), n_tokens as i64, ys.as_mut_ptr()) })?;
        Ok((CpuStorage::F32(ys), layout.shape().clone()))
    }
}

impl Module for HipSparseMoe {
    /// `[b, seq, hidden]` in, the same shape out (quantized_llama.rs:151, 205).
    fn forward(&self, xs: &Tensor) -> Result<Tensor> {
        xs.contiguous()?.apply_op1_no_bwd(self)
    }
}

impl Drop for HipSparseMoe {
    fn drop(&mut self) {
        unsafe { ffi::moe_layer_destroy(self.handle) }
    }
}

// ------------------------------------------------------------------------------------------------ projections

/// One quantized `[n, k]` matrix resident on the GPU: `xs . W^T`, the `QMatMul::QTensor` arm.
pub struct HipQMatMul {
    handle: *mut ffi::MoeQLinear,
    n: usize,
    k: usize,
}
unsafe impl Send for HipQMatMul {}
unsafe impl Sync for HipQMatMul {}

impl HipQMatMul {
    /// `QMatMul::from_qtensor` (quantized/mod.rs:445-447) for a quantized CPU tensor of rank 2.
    pub fn from_qtensor(w: &QTensor) -> Result<Self> {
        let (n, k) = w.shape().dims2()?;
        let data = w.data()?;   // kept alive across the call
        let mut handle = std::ptr::null_mut();
        check(unsafe { ffi::moe_qlinear_create(ggml_id(w.dtype())?, data.as_ptr() as *const c_void, n as i64, k as i64, &mut handle) })?;
        Ok(Self { handle, n, k })
    }

    /// `QMatMul::from_qtensor(ct.tensor(reader, name, device)?)` (quantized_llama.rs:533-547) read from the file.
    pub fn from_gguf<P: AsRef<Path>>(path: P, tensor_name: &str) -> Result<Self> {
        let file = GgufFile::open(path)?;
        let name = CString::new(tensor_name).map_err(candle::Error::wrap)?;
        let mut handle = std::ptr::null_mut();
        check(unsafe { ffi::moe_qlinear_create_from_gguf(file.0, name.as_ptr(), &mut handle) })?;
        let (mut n, mut k, mut dt) = (0i64, 0i64, 0i32);
        check(unsafe { ffi::moe_qlinear_shape(handle, &mut n, &mut k, &mut dt) })?;
        Ok(Self { handle, n: n as usize, k: k as usize })
    }

    /// `QMatMul::dequantize` of the resident copy: f32 `[n, k]`.
    pub fn dequantize(&self) -> Result<Tensor> {
        let mut out = vec![0f32; self.n * self.k];
        check(unsafe { ffi::moe_qlinear_dequantize(self.handle, out.as_mut_ptr(), out.len() as i64) })?;
        Tensor::from_vec(out, (self.n, self.k), &candle::Device::Cpu)
    }
}

impl CustomOp1 for HipQMatMul {
    fn name(&self) -> &'static str {
        "qmatmul"
    }

    /// Same checks and shapes as `QTensor::cpu_fwd` (quantized/mod.rs:475-506).
    fn cpu_fwd(&self, storage: &CpuStorage, layout: &Layout) -> Result<(CpuStorage, Shape)> {
        let xs = contiguous_f32(storage, layout, "qmatmul")?;
        let src_shape = layout.shape();
        if src_shape.rank() < 2 {
            bail!("input tensor has only one dimension {layout:?}")
        }
        let mut dst_shape = src_shape.dims().to_vec();
        let last_k = dst_shape.pop().unwrap_or(0);
        if last_k != self.k {
            bail!("input tensor {layout:?} incompatible with [{}, {}]", self.n, self.k)
        }
        dst_shape.push(self.n);
        let dst_shape = Shape::from(dst_shape);
        let m = xs.len() / self.k;
        let mut ys = vec![0f32; dst_shape.elem_count()];
        check(unsafe { ffi::moe_qlinear_forward(self.handle, xs.as_ptr(), m as i64, ys.as_mut_ptr()) })?;
        Ok((CpuStorage::F32(ys), dst_shape))
    }
}

impl Module for HipQMatMul {
    fn forward(&self, xs: &Tensor) -> Result<Tensor> {
        xs.apply_op1_no_bwd(self)
    }
}

impl Drop for HipQMatMul {
    fn drop(&mut self) {
        unsafe { ffi::moe_qlinear_destroy(self.handle) }
    }
}

// ------------------------------------------------------------------------------------------------ rms-norm

/// `RmsNorm` (quantized_nn.rs:100-126): the sum of squares is taken left to right as `candle_nn::ops::rms_norm`
/// takes it (candle-nn/src/ops.rs:504-515), so the result equals the CPU one bit for bit.
pub struct HipRmsNorm {
    weight: Vec<f32>,
    eps: f32,
}

impl HipRmsNorm {
    pub fn from_qtensor(weight: QTensor, eps: f64) -> Result<Self> {
        let weight = f32_vec(&weight.dequantize(&candle::Device::Cpu)?)?;
        Ok(Self { weight, eps: eps as f32 })
    }
}

impl CustomOp1 for HipRmsNorm {
    fn name(&self) -> &'static str {
        "hip-rms-norm"
    }

    fn cpu_fwd(&self, storage: &CpuStorage, layout: &Layout) -> Result<(CpuStorage, Shape)> {
        let xs = contiguous_f32(storage, layout, "hip-rms-norm")?;
        let hidden = self.weight.len();
        if layout.shape().dims().last().copied() != Some(hidden) {
            bail!("hip-rms-norm: input {:?} does not end in {hidden}", layout.shape())
        }
        let mut ys = vec![0f32; xs.len()];
        check(unsafe { ffi::moe_rms_norm(xs.as_ptr(), self.weight.as_ptr(), self.eps, (xs.len() / hidden) as i64, hidden as i64, ys.as_mut_ptr()) })?;
        Ok((CpuStorage::F32(ys), layout.shape().clone()))
    }
}

impl Module for HipRmsNorm {
    fn forward(&self, xs: &Tensor) -> Result<Tensor> {
        xs.contiguous()?.apply_op1_no_bwd(self)
    }
}

// ------------------------------------------------------------------------------------------------ GGUF handle

struct GgufFile(*mut ffi::MoeGguf);

impl GgufFile {
    fn open<P: AsRef<Path>>(path: P) -> Result<Self> {
        let p = path.as_ref().to_str().ok_or_else(|| candle::Error::Msg("path is not valid UTF-8".to_string()))?;
        let c = CString::new(p).map_err(candle::Error::wrap)?;
        let mut h = std::ptr::null_mut();
        check(unsafe { ffi::moe_gguf_open(c.as_ptr() as *const c_char, &mut h) })?;
        Ok(Self(h))
    }
}

impl Drop for GgufFile {
    fn drop(&mut self) {
        unsafe { ffi::moe_gguf_close(self.0) }
    }
}
