//! `hip` op back end for rust-model-inference: binds librmi_hip.so (C ABI in
//! include/rmi_hip.h) and implements the crate's existing `Kernel` and `Layer`
//! traits on top of it.
//!
//! NOT COMPILED in the environment this back end was built in (no Rust
//! toolchain there); it is the binding a maintainer drops into the crate as
//! `src/hip.rs` behind `--features hip`, and it is kept thin so that it can be
//! reviewed by eye: every method is one FFI call.
//!
//! Hook points in the crate:
//!   * `QuantizedTensor::into_kernel` (src/ops/kernel/quantized_tensor.rs:167-190):
//!     when `ops::hip_enabled()` return `Box::new(HipKernel::upload(..))` for
//!     `Q8_0` / `Q4_K` / `Q6_K` instead of `Q8Kernel` / `Q4_KKernel` / `Q6_KKernel`;
//!   * `ops::enable_gpu` / the lazy context of src/ops/float.rs:44-58: call
//!     `hip::init(0)`; on `Err` print and stay on the CPU kernels, as today;
//!   * `matmul_q8_0_quantized_range` (src/ops/kernel/q8_0/dispatch.rs:36-52) is NOT
//!     hooked: its weight argument is a borrowed byte slice with no handle.

use std::ffi::{c_char, c_int, c_void, CStr};

use crate::core::traits::{ExecContext, Layer};
use crate::ops::kernel::Kernel;
use crate::ops::quant::BlockQ8K;

#[repr(C)]
pub struct RmiHipWeight {
    _private: [u8; 0],
}

#[link(name = "rmi_hip")]
extern "C" {
    fn rmi_hip_init(device: c_int) -> c_int;
    fn rmi_hip_last_error() -> *const c_char;
    fn rmi_hip_upload_q8_0(blocks: *const u8, nbytes: usize, n_in: u32, n_out: u32) -> *mut RmiHipWeight;
    fn rmi_hip_upload_q4_k(blocks: *const u8, nbytes: usize, n_in: u32, n_out: u32) -> *mut RmiHipWeight;
    fn rmi_hip_upload_q4_0(blocks: *const u8, nbytes: usize, n_in: u32, n_out: u32) -> *mut RmiHipWeight;
    fn rmi_hip_upload_q6_k(blocks: *const u8, nbytes: usize, n_in: u32, n_out: u32) -> *mut RmiHipWeight;
    fn rmi_hip_fuse_vstack(a: *const RmiHipWeight, b: *const RmiHipWeight) -> *mut RmiHipWeight;
    fn rmi_hip_free_weight(w: *mut RmiHipWeight);
    fn rmi_hip_q8_0_forward_prequantized(
        w: *const RmiHipWeight, input_q8: *const u8, input_scales: *const f32, output: *mut f32,
        n_in: u32, n_out: u32, ith: u32, nth: u32,
    ) -> c_int;
    fn rmi_hip_q8_0_forward_batched(
        w: *const RmiHipWeight, input: *const f32, output: *mut f32, n_in: u32, n_out: u32, n_tokens: u32,
        rounding: c_int,
    ) -> c_int;
    fn rmi_hip_set_forward_batched_mode(mode: c_int) -> c_int;
    fn rmi_hip_q8_0_forward_batched_neon(
        w: *const RmiHipWeight, input: *const f32, output: *mut f32, n_in: u32, n_out: u32, n_tokens: u32,
        rounding: c_int,
    ) -> c_int;
    fn rmi_hip_q4_k_forward_batched_mfma(
        w: *const RmiHipWeight, input: *const f32, output: *mut f32, n_in: u32, n_out: u32, n_tokens: u32,
    ) -> c_int;
    fn rmi_hip_q4_k_forward_prepared(
        w: *const RmiHipWeight, d: *const f32, qs: *const i8, bsums: *const i16, output: *mut f32,
        n_in: u32, n_out: u32, ith: u32, nth: u32,
    ) -> c_int;
    fn rmi_hip_q4_k_forward_batched(
        w: *const RmiHipWeight, input: *const f32, output: *mut f32, n_in: u32, n_out: u32, n_tokens: u32,
    ) -> c_int;
    fn rmi_hip_q4_k_forward_prequantized(
        w: *const RmiHipWeight, input_q8: *const u8, input_scales: *const f32, output: *mut f32,
        n_in: u32, n_out: u32, ith: u32, nth: u32,
    ) -> c_int;
    fn rmi_hip_q4_0_forward_prequantized(
        w: *const RmiHipWeight, input_q8: *const u8, input_scales: *const f32, output: *mut f32,
        n_in: u32, n_out: u32, ith: u32, nth: u32,
    ) -> c_int;
    fn rmi_hip_q4_0_forward_batched(
        w: *const RmiHipWeight, input: *const f32, output: *mut f32, n_in: u32, n_out: u32, n_tokens: u32,
        rounding: c_int,
    ) -> c_int;
    fn rmi_hip_q6_k_forward_prepared(
        w: *const RmiHipWeight, d: *const f32, qs: *const i8, bsums: *const i16, output: *mut f32,
        n_in: u32, n_out: u32, ith: u32, nth: u32,
    ) -> c_int;
    fn rmi_hip_q6_k_forward_batched(
        w: *const RmiHipWeight, input: *const f32, output: *mut f32, n_in: u32, n_out: u32, n_tokens: u32,
    ) -> c_int;
    fn rmi_hip_q6_k_forward_prequantized(
        w: *const RmiHipWeight, input_q8: *const u8, input_scales: *const f32, output: *mut f32,
        n_in: u32, n_out: u32, ith: u32, nth: u32,
    ) -> c_int;
    fn rmi_hip_quantized_linear_forward(
        w: *const RmiHipWeight, input: *const f32, output: *mut f32, in_features: u32, out_features: u32,
    ) -> c_int;
}

const ROUND_TIES_EVEN: c_int = 1; // what quantize_q8_0_into does on x86-64 (src/ops/quant/q8_0.rs:5-12)

fn last_error() -> String {
    unsafe { CStr::from_ptr(rmi_hip_last_error()).to_string_lossy().into_owned() }
}

/// `Err` means "stay on the CPU kernels" (src/ops/float.rs:51-57).
pub fn init(device: i32) -> Result<(), String> {
    if unsafe { rmi_hip_init(device) } == 0 { Ok(()) } else { Err(last_error()) }
}

/// How `Kernel::forward_batched` of the Q8_0 and Q4_K kernels multiplies a batch, for the whole process
/// (`rmi_hip_set_forward_batched_mode`): the x86-64 kernels' bits for every token (the default), the aarch64
/// kernel's bits, or the fastest kernel per product within the crate's own tolerance (exact integer block dots,
/// f32 sums within 1e-4 + 1e-4 |ref|).  Chosen once at start-up; no call site changes.
#[derive(Clone, Copy, PartialEq)]
pub enum BatchedMode { X86Order = 0, Aarch64Order = 1, Fast = 2 }

pub fn set_forward_batched_mode(mode: BatchedMode) -> Result<(), String> {
    if unsafe { rmi_hip_set_forward_batched_mode(mode as c_int) } == 0 { Ok(()) } else { Err(last_error()) }
}

#[derive(Clone, Copy, PartialEq)]
enum Dtype { Q8_0, Q4_0, Q4K, Q6K }

/// A weight resident in HBM.  `Kernel: Send + Sync`: the library gives every
/// calling thread its own stream and staging, so `&self` calls may overlap.
pub struct HipKernel {
    handle: *mut RmiHipWeight,
    dtype: Dtype,
}
unsafe impl Send for HipKernel {}
unsafe impl Sync for HipKernel {}

impl HipKernel {
    pub fn upload_q8_0(weight: &[u8], n_in: usize, n_out: usize) -> Result<Self, String> {
        let h = unsafe { rmi_hip_upload_q8_0(weight.as_ptr(), weight.len(), n_in as u32, n_out as u32) };
        if h.is_null() { Err(last_error()) } else { Ok(Self { handle: h, dtype: Dtype::Q8_0 }) }
    }
    pub fn upload_q4_k(weight: &[u8], n_in: usize, n_out: usize) -> Result<Self, String> {
        let h = unsafe { rmi_hip_upload_q4_k(weight.as_ptr(), weight.len(), n_in as u32, n_out as u32) };
        if h.is_null() { Err(last_error()) } else { Ok(Self { handle: h, dtype: Dtype::Q4K }) }
    }
    pub fn upload_q4_0(weight: &[u8], n_in: usize, n_out: usize) -> Result<Self, String> {
        let h = unsafe { rmi_hip_upload_q4_0(weight.as_ptr(), weight.len(), n_in as u32, n_out as u32) };
        if h.is_null() { Err(last_error()) } else { Ok(Self { handle: h, dtype: Dtype::Q4_0 }) }
    }
    pub fn upload_q6_k(weight: &[u8], n_in: usize, n_out: usize) -> Result<Self, String> {
        let h = unsafe { rmi_hip_upload_q6_k(weight.as_ptr(), weight.len(), n_in as u32, n_out as u32) };
        if h.is_null() { Err(last_error()) } else { Ok(Self { handle: h, dtype: Dtype::Q6K }) }
    }
    /// `QTensorOwned::fuse_vstack` (src/ops/kernel/qtensor_owned.rs:138-164)
    pub fn fuse_vstack(a: &Self, b: &Self) -> Option<Self> {
        let h = unsafe { rmi_hip_fuse_vstack(a.handle, b.handle) };
        if h.is_null() { None } else { Some(Self { handle: h, dtype: a.dtype }) }
    }
}

impl Drop for HipKernel {
    fn drop(&mut self) { unsafe { rmi_hip_free_weight(self.handle) } }
}

fn expect_ok(rc: c_int) {
    if rc != 0 { panic!("GPU matmul failed: {}", last_error()); } // dispatch.rs:47-48
}

impl Kernel for HipKernel {
    fn forward_prequantized(
        &self, input_q8: &[u8], input_scales: &[f32], output: &mut [f32],
        n_in: usize, n_out: usize, ith: usize, nth: usize,
    ) {
        let rc = unsafe {
            match self.dtype {
                Dtype::Q8_0 => rmi_hip_q8_0_forward_prequantized(
                    self.handle, input_q8.as_ptr(), input_scales.as_ptr(), output.as_mut_ptr(),
                    n_in as u32, n_out as u32, ith as u32, nth as u32),
                Dtype::Q4_0 => rmi_hip_q4_0_forward_prequantized(
                    self.handle, input_q8.as_ptr(), input_scales.as_ptr(), output.as_mut_ptr(),
                    n_in as u32, n_out as u32, ith as u32, nth as u32),
                Dtype::Q4K => rmi_hip_q4_k_forward_prequantized(
                    self.handle, input_q8.as_ptr(), input_scales.as_ptr(), output.as_mut_ptr(),
                    n_in as u32, n_out as u32, ith as u32, nth as u32),
                Dtype::Q6K => rmi_hip_q6_k_forward_prequantized(
                    self.handle, input_q8.as_ptr(), input_scales.as_ptr(), output.as_mut_ptr(),
                    n_in as u32, n_out as u32, ith as u32, nth as u32),
            }
        };
        expect_ok(rc);
    }

    fn forward_prepared(
        &self, input_f32: &[f32], input_q8: &[u8], input_scales: &[f32], q8_k: Option<&[BlockQ8K]>,
        output: &mut [f32], n_in: usize, n_out: usize, ith: usize, nth: usize,
    ) {
        if self.dtype == Dtype::Q8_0 || self.dtype == Dtype::Q4_0 {
            return self.forward_prequantized(input_q8, input_scales, output, n_in, n_out, ith, nth);
        }
        // BlockQ8K has no repr(C) (src/ops/quant/mod.rs:35-40): pass three arrays.
        let owned;
        let blocks: &[BlockQ8K] = match q8_k {
            Some(b) => b,
            None => { owned = crate::ops::quant::quantize_row_q8_k(&input_f32[..n_in]); &owned } // q4_k.rs:77-84, q6_k.rs:63-69
        };
        let d: Vec<f32> = blocks.iter().map(|b| b.d).collect();
        let qs: Vec<i8> = blocks.iter().flat_map(|b| b.qs.iter().copied()).collect();
        let bs: Vec<i16> = blocks.iter().flat_map(|b| b.bsums.iter().copied()).collect();
        let prepared = if self.dtype == Dtype::Q6K { rmi_hip_q6_k_forward_prepared } else { rmi_hip_q4_k_forward_prepared };
        expect_ok(unsafe {
            prepared(self.handle, d.as_ptr(), qs.as_ptr(), bs.as_ptr(), output.as_mut_ptr(),
                     n_in as u32, n_out as u32, ith as u32, nth as u32)
        });
    }

    fn forward(&self, input: &[f32], output: &mut [f32], n_in: usize, n_out: usize) {
        self.forward_batched(&input[..n_in], &mut output[..n_out], n_in, n_out);
    }

    fn forward_batched(&self, input: &[f32], output: &mut [f32], n_in: usize, n_out: usize) {
        let n_tokens = (input.len() / n_in) as u32;
        expect_ok(unsafe {
            match self.dtype {
                Dtype::Q8_0 => rmi_hip_q8_0_forward_batched(self.handle, input.as_ptr(), output.as_mut_ptr(),
                                                            n_in as u32, n_out as u32, n_tokens, ROUND_TIES_EVEN),
                Dtype::Q4_0 => rmi_hip_q4_0_forward_batched(self.handle, input.as_ptr(), output.as_mut_ptr(),
                                                            n_in as u32, n_out as u32, n_tokens, ROUND_TIES_EVEN),
                Dtype::Q4K => rmi_hip_q4_k_forward_batched(self.handle, input.as_ptr(), output.as_mut_ptr(),
                                                           n_in as u32, n_out as u32, n_tokens),
                Dtype::Q6K => rmi_hip_q6_k_forward_batched(self.handle, input.as_ptr(), output.as_mut_ptr(),
                                                           n_in as u32, n_out as u32, n_tokens),
            }
        });
    }
}

impl HipKernel {
    /// Prefill: `forward_batched` on the int8 matrix cores.  Q8_0 results follow the aarch64 kernel's order
    /// (neon.rs:49-73), Q4_K results one f32 chain per output; both within 1e-4 + 1e-4*|ref| of `forward_batched`,
    /// which stays bit-identical to the x86-64 kernels for every token count.
    pub fn forward_batched_matrix_cores(&self, input: &[f32], output: &mut [f32], n_in: usize, n_out: usize) {
        let n_tokens = (input.len() / n_in) as u32;
        match self.dtype {
            Dtype::Q8_0 => expect_ok(unsafe {
                rmi_hip_q8_0_forward_batched_neon(self.handle, input.as_ptr(), output.as_mut_ptr(), n_in as u32,
                                                  n_out as u32, n_tokens, ROUND_TIES_EVEN)
            }),
            Dtype::Q4K => expect_ok(unsafe {
                rmi_hip_q4_k_forward_batched_mfma(self.handle, input.as_ptr(), output.as_mut_ptr(), n_in as u32,
                                                  n_out as u32, n_tokens)
            }),
            _ => self.forward_batched(input, output, n_in, n_out),
        }
    }
}

/// `QuantizedLinear` (src/core/model.rs:12-104) on the GPU: same constructor
/// arguments, `ctx.scratch` is not used (the weight is dequantised in registers).
pub struct HipLinear<'a> {
    kernel: HipKernel,
    in_features: usize,
    out_features: usize,
    layer_name: &'a str,
}

impl<'a> HipLinear<'a> {
    pub fn from_weight_slice(weight: &[u8], _bias: Option<&[u8]>, in_features: usize, out_features: usize,
                             name: &'a str) -> Result<Self, String> {
        Ok(Self { kernel: HipKernel::upload_q4_k(weight, in_features, out_features)?, in_features, out_features,
                  layer_name: name })
    }
}

impl<'a> Layer for HipLinear<'a> {
    fn forward(&self, input: &[f32], output: &mut [f32], _ctx: &mut ExecContext) {
        expect_ok(unsafe {
            rmi_hip_quantized_linear_forward(self.kernel.handle, input.as_ptr(), output.as_mut_ptr(),
                                             self.in_features as u32, self.out_features as u32)
        });
    }
    fn input_dim(&self) -> usize { self.in_features }
    fn output_dim(&self) -> usize { self.out_features }
    fn name(&self) -> &str { self.layer_name }
}

// ---------------------------------------------------------------- device-resident decode
//
// `Qwen3Session::generate_inner` (src/models/qwen3.rs:581-1158) with every tensor in HBM between two
// token ids.  The two structs mirror rmi_hip_qwen3_config / rmi_hip_qwen3_weights of rmi_hip.h.

#[repr(C)]
pub struct RmiQwen3Config {
    pub n_embd: u32, pub n_layer: u32, pub n_head: u32, pub n_head_kv: u32, pub head_dim_k: u32, pub head_dim_v: u32,
    pub n_ff: u32, pub vocab: u32, pub capacity: u32,
    pub eps: f32, pub freq_base: f32,
    pub has_qk_norm: i32, pub rounding: i32,
}

#[repr(C)]
pub struct RmiQwen3Weights {
    pub token_embd: *const u8, pub output: *const u8, pub output_norm: *const f32,
    pub attn_norm: *const *const f32, pub ffn_norm: *const *const f32,
    pub q_norm: *const *const f32, pub k_norm: *const *const f32,
    pub wq: *const *const u8, pub wk: *const *const u8, pub wv: *const *const u8, pub wo: *const *const u8,
    pub w_gate: *const *const u8, pub w_up: *const *const u8, pub w_down: *const *const u8,
}

extern "C" {
    fn rmi_hip_qwen3_create(cfg: *const RmiQwen3Config, weights: *const RmiQwen3Weights) -> *mut c_void;
    fn rmi_hip_qwen3_destroy(s: *mut c_void);
    fn rmi_hip_qwen3_generate(s: *mut c_void, prompt: *const u32, n_prompt: u32, max_new: u32, generated: *mut u32,
                              step_argmax: *mut u32, step_top2: *mut f32, dump_steps: *const u32, n_dump: u32,
                              dump_logits: *mut f32, seconds: *mut f64) -> c_int;
}

extern "C" {
    fn rmi_hip_gguf_open(path: *const std::os::raw::c_char) -> *mut c_void;
    fn rmi_hip_gguf_close(g: *mut c_void);
    fn rmi_hip_gguf_meta_u64(g: *const c_void, key: *const std::os::raw::c_char, out: *mut u64) -> c_int;
    fn rmi_hip_gguf_meta_f64(g: *const c_void, key: *const std::os::raw::c_char, out: *mut f64) -> c_int;
    fn rmi_hip_gguf_upload_stack(g: *const c_void, names: *const *const std::os::raw::c_char, n: c_int)
                                 -> *mut RmiHipWeight;
    fn rmi_hip_weight_dtype(w: *const RmiHipWeight) -> c_int;
    fn rmi_hip_qwen3_create_from_gguf(g: *const c_void, capacity: u32, rounding: c_int) -> *mut c_void;
}

/// The file as the library maps and parses it (`GGUFLoader::from_file`, src/core/loader.rs:211-320, with the
/// reference's error messages).  A crate that keeps its own `GGUFLoader` for tokenizer metadata opens this one
/// next to it for the weights: tensor bytes then go from the page cache to HBM without passing through a slice.
pub struct HipGguf { handle: *mut c_void }
unsafe impl Send for HipGguf {}

impl HipGguf {
    pub fn from_file(path: &str) -> Result<Self, String> {
        let c = std::ffi::CString::new(path).map_err(|e| e.to_string())?;
        let handle = unsafe { rmi_hip_gguf_open(c.as_ptr()) };
        if handle.is_null() { Err(last_error()) } else { Ok(Self { handle }) }
    }
    /// `metadata(key).and_then(MetaValue::to_u64)`
    pub fn to_u64(&self, key: &str) -> Option<u64> {
        let c = std::ffi::CString::new(key).ok()?;
        let mut v = 0u64;
        if unsafe { rmi_hip_gguf_meta_u64(self.handle, c.as_ptr(), &mut v) } != 0 { Some(v) } else { None }
    }
    /// `metadata(key).and_then(MetaValue::to_f64)`
    pub fn to_f64(&self, key: &str) -> Option<f64> {
        let c = std::ffi::CString::new(key).ok()?;
        let mut v = 0f64;
        if unsafe { rmi_hip_gguf_meta_f64(self.handle, c.as_ptr(), &mut v) } != 0 { Some(v) } else { None }
    }
    /// One matrix of the file, or several stacked row-wise (`[q ; k ; v]`, `[gate ; up]`), as a kernel in HBM.
    pub fn kernel(&self, names: &[&str]) -> Result<HipKernel, String> {
        let owned: Vec<std::ffi::CString> =
            names.iter().map(|n| std::ffi::CString::new(*n).map_err(|e| e.to_string())).collect::<Result<_, _>>()?;
        let ptrs: Vec<*const std::os::raw::c_char> = owned.iter().map(|c| c.as_ptr()).collect();
        let h = unsafe { rmi_hip_gguf_upload_stack(self.handle, ptrs.as_ptr(), ptrs.len() as c_int) };
        if h.is_null() { return Err(last_error()); }
        let dtype = match unsafe { rmi_hip_weight_dtype(h) } {
            2 => Dtype::Q4_0,
            8 => Dtype::Q8_0,
            12 => Dtype::Q4K,
            _ => Dtype::Q6K,
        };
        Ok(HipKernel { handle: h, dtype })
    }
    /// `Qwen3Model::from_source` + `Qwen3Session::new` (src/models/qwen3.rs:262-349) on the device.
    pub fn qwen3_session(&self, capacity: usize) -> Result<HipQwen3Session, String> {
        let handle = unsafe { rmi_hip_qwen3_create_from_gguf(self.handle, capacity as u32, 1) };
        if handle.is_null() { Err(last_error()) } else { Ok(HipQwen3Session { handle }) }
    }
}

impl Drop for HipGguf {
    fn drop(&mut self) { unsafe { rmi_hip_gguf_close(self.handle) } }
}

/// Owns the HBM copy of a model and its KV cache.  Built from the tensors `Qwen3Model::from_gguf`
/// (src/models/qwen3.rs:263-420) borrows from the mmap; the slices may be dropped after `new`.
pub struct HipQwen3Session { handle: *mut c_void }
unsafe impl Send for HipQwen3Session {}

impl HipQwen3Session {
    pub fn new(cfg: &RmiQwen3Config, weights: &RmiQwen3Weights) -> Result<Self, String> {
        let handle = unsafe { rmi_hip_qwen3_create(cfg, weights) };
        if handle.is_null() { Err(last_error()) } else { Ok(Self { handle }) }
    }

    /// Greedy generation, the prompt fed one token per step as `generate_inner` does.
    pub fn generate(&mut self, prompt: &[u32], max_new: usize) -> Result<Vec<u32>, String> {
        let mut out = vec![0u32; max_new];
        let n = unsafe {
            rmi_hip_qwen3_generate(self.handle, prompt.as_ptr(), prompt.len() as u32, max_new as u32, out.as_mut_ptr(),
                                   std::ptr::null_mut(), std::ptr::null_mut(), std::ptr::null(), 0,
                                   std::ptr::null_mut(), std::ptr::null_mut())
        };
        if n < 0 { return Err(last_error()); }
        out.truncate(n as usize);
        Ok(out)
    }
}

impl Drop for HipQwen3Session {
    fn drop(&mut self) { unsafe { rmi_hip_qwen3_destroy(self.handle) } }
}
