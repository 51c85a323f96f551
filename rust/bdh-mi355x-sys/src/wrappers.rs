//! Safe wrappers with the reference crate's signatures over a Burn backend whose tensors carry HIP device
//! pointers.  A maintainer routes `FusedKernelConfig.enabled` (src/model/bdh.rs:332,337,361;
//! src/model/attention.rs:143) to these.  Not compiled in this repository's environment.
use std::ffi::CStr;
use std::os::raw::c_void;

use burn::tensor::{backend::Backend, Int, Tensor};

use crate::*;

/// Backend extension: float tensors expose a device pointer, the device a HIP stream.
pub trait HipPointers: Backend {
    fn device_ptr<const D: usize>(t: &Tensor<Self, D>) -> *mut f32;
    fn int_device_ptr<const D: usize>(t: &Tensor<Self, D, Int>) -> *mut i64;
    fn hip_stream(device: &Self::Device) -> *mut c_void;
    fn device_index(device: &Self::Device) -> i32;
}

/// src/positional.rs:8-15
#[derive(Clone, Copy, PartialEq, Eq)]
pub enum RotaryEmbedding {
    Rope = 0,
    Alibi = 1,
    Pope = 2,
}

/// Owns a `bdh_ctx`; one per (device, stream), not re-entrant.
pub struct Ctx {
    raw: *mut bdh_ctx,
}

impl Ctx {
    pub fn new<B: HipPointers>(device: &B::Device) -> Self {
        let mut raw = std::ptr::null_mut();
        let rc = unsafe { bdh_ctx_create(B::device_index(device), B::hip_stream(device), &mut raw) };
        assert_eq!(rc, BDH_OK, "bdh_ctx_create failed: is a HIP device present?");
        Ctx { raw }
    }
    pub fn last_error(&self) -> String {
        unsafe { CStr::from_ptr(bdh_last_error(self.raw)) }.to_string_lossy().into_owned()
    }
    /// the reference panics on contract violations (src/model/bdh.rs:314-318); so does the wrapper
    fn check(&self, rc: i32) {
        assert_eq!(rc, BDH_OK, "{}", self.last_error());
    }
}

impl Drop for Ctx {
    fn drop(&mut self) {
        unsafe { bdh_ctx_destroy(self.raw) };
    }
}

/// src/model/state.rs:5-15
pub struct LayerState<B: Backend> {
    pub rho: Option<Tensor<B, 4>>,
}

/// drop-in for kernel::relu_lowrank::fused_forward (src/kernel/relu_lowrank.rs:7-37);
/// `active_blocks` = BlockPattern1d as one byte per latent block (src/kernel/block_sparse.rs:11-63), None = dense
pub fn relu_lowrank_fused_forward<B: HipPointers>(ctx: &Ctx, input: Tensor<B, 4>, weight: Tensor<B, 4>,
    bias: Option<Tensor<B, 3>>, threshold: f32, block_size: usize, active_blocks: Option<&[u8]>) -> Tensor<B, 4> {
    let [b, h_in, t, d] = input.dims();
    let [_, h, _, n] = weight.dims();
    let out = Tensor::<B, 4>::empty([b, h, t, n], &input.device());
    let (blocks_ptr, n_blocks) = active_blocks.map_or((std::ptr::null(), 0), |a| (a.as_ptr(), a.len() as i32));
    let bias_ptr = bias.as_ref().map_or(std::ptr::null(), |t| B::device_ptr(t) as *const f32);
    ctx.check(unsafe {
        bdh_relu_lowrank(ctx.raw, b as i32, h_in as i32, t as i32, d as i32, h as i32, n as i32,
            B::device_ptr(&input), B::device_ptr(&weight), bias_ptr, threshold, block_size as i32, blocks_ptr,
            n_blocks, std::ptr::null(), B::device_ptr(&out))
    });
    out
}

/// drop-in for BDH::recurrent_attention (src/model/bdh.rs:258-307, the rotate of :265 included)
pub fn recurrent_attention<B: HipPointers>(ctx: &Ctx, query: Tensor<B, 4>, value: Tensor<B, 4>,
    freqs: &Tensor<B, 4>, layer_state: &mut LayerState<B>, position: usize, rotary: RotaryEmbedding) -> Tensor<B, 4> {
    let [b, h, t, n] = query.dims();
    let d = value.dims()[3];
    let nq = if rotary == RotaryEmbedding::Pope { 2 * n } else { n };
    // zero state on first use or shape change (src/model/bdh.rs:274-284)
    let rho = match layer_state.rho.take() {
        Some(r) if r.dims() == [b, h, nq, d] => r,
        _ => Tensor::<B, 4>::zeros([b, h, nq, d], &value.device()),
    };
    let out = Tensor::<B, 4>::empty([b, h, t, d], &value.device());
    ctx.check(unsafe {
        bdh_recurrent_attention(ctx.raw, b as i32, h as i32, t as i32, n as i32, d as i32, rotary as i32,
            B::device_ptr(&query), B::device_ptr(&value), B::device_ptr(freqs), position as i64, std::ptr::null(),
            std::ptr::null(), B::device_ptr(&rho) as *mut c_void, BDH_F32, B::device_ptr(&out),
            std::ptr::null_mut(), std::ptr::null_mut())
    });
    layer_state.rho = Some(rho); // moved back (src/model/bdh.rs:304)
    out
}

/// drop-in for kernel::linear_attention::fused_state_aligned (src/kernel/linear_attention.rs:11-115);
/// `block_pairs` = the active (row, col) time blocks of a sparse BlockPattern2d, None = dense (col <= row)
pub fn fused_state_aligned<B: HipPointers>(ctx: &Ctx, query: Tensor<B, 4>, value: Tensor<B, 4>, freqs: Tensor<B, 4>,
    alibi_slopes: Option<&[f32]>, block_size: usize, block_pairs: Option<&[i32]>, rotary: RotaryEmbedding)
    -> Tensor<B, 4> {
    let [b, h, t, n] = query.dims();
    let dv = value.dims()[3];
    let out = Tensor::<B, 4>::empty([b, h, t, dv], &value.device());
    let (pairs_ptr, n_pairs) = block_pairs.map_or((std::ptr::null(), 0), |p| (p.as_ptr(), (p.len() / 2) as i32));
    ctx.check(unsafe {
        bdh_fused_state_aligned(ctx.raw, b as i32, h as i32, t as i32, n as i32, dv as i32, B::device_ptr(&query),
            B::device_ptr(&value), B::device_ptr(&freqs), alibi_slopes.map_or(std::ptr::null(), |s| s.as_ptr()),
            block_size as i32, pairs_ptr, n_pairs, rotary as i32, 1, B::device_ptr(&out))
    });
    out
}

/// drop-in for BDH::forward_with_state (src/model/bdh.rs:309-450): `rho` holds all layers [L,B,h,Nq,d]
pub fn forward_with_state<B: HipPointers>(ctx: &Ctx, model: *mut bdh_model, tokens: Tensor<B, 2, Int>,
    rho: &Tensor<B, 5>, position: &mut usize, vocab: usize) -> Tensor<B, 3> {
    let [b, t] = tokens.dims();
    let logits = Tensor::<B, 3>::empty([b, t, vocab], &tokens.device());
    ctx.check(unsafe {
        bdh_model_forward(model, B::int_device_ptr(&tokens), b as i32, t as i32, B::device_ptr(rho) as *mut c_void,
            BDH_F32, *position as i64, B::device_ptr(&logits), std::ptr::null_mut(), std::ptr::null_mut())
    });
    *position = position.saturating_add(t); // src/model/bdh.rs:445
    logits
}
