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

/// src/model/state.rs:10-15: one independent state tensor per layer and the shared position
pub struct ModelState<B: Backend> {
    pub layers: Vec<LayerState<B>>,
    pub position: usize,
}

impl<B: Backend> ModelState<B> {
    /// src/model/state.rs:27-38
    pub fn new(num_layers: usize) -> Self {
        ModelState { layers: (0..num_layers).map(|_| LayerState { rho: None }).collect(), position: 0 }
    }
    /// src/model/state.rs:40-45
    pub fn reset(&mut self) {
        for layer in self.layers.iter_mut() {
            layer.rho = None;
        }
        self.position = 0;
    }
}

/// The model's shapes as BDHConfig gives them (src/model/config.rs:113-164)
#[derive(Clone, Copy)]
pub struct ModelDims {
    pub n_layer: usize,
    pub n_embd: usize,
    pub n_head: usize,
    pub latent: usize,
    pub vocab: usize,
    pub rotary: RotaryEmbedding,
    pub rope_theta: f32,
    pub relu_threshold: f32,
}

/// Owns a `bdh_model` (destroyed on drop) together with the parameter tensors it points into and the context it
/// launches on: the inference half of BDH<B> (src/model/bdh.rs:27-33).
pub struct Model<B: HipPointers> {
    raw: *mut bdh_model,
    ctx: Ctx,
    dims: ModelDims,
    // the record order of the reference module; kept alive because the library holds their device pointers
    _embed: Tensor<B, 2>,
    _encoder: Tensor<B, 3>,
    _encoder_v: Tensor<B, 3>,
    _decoder: Tensor<B, 2>,
    _lm_head: Tensor<B, 2>,
}

impl<B: HipPointers> Model<B> {
    /// BDH::new as far as inference needs it (src/model/bdh.rs:37-84): `embed [V,d]`, `encoder`/`encoder_v [h,d,N]`,
    /// `decoder [h*N,d]`, `lm_head [d,V]` are the Param values of the reference module (`.val()`, bdh.rs:324-331).
    pub fn new(device: &B::Device, dims: ModelDims, embed: Tensor<B, 2>, encoder: Tensor<B, 3>,
        encoder_v: Tensor<B, 3>, decoder: Tensor<B, 2>, lm_head: Tensor<B, 2>, alibi_slopes: Option<&[f32]>) -> Self {
        let ctx = Ctx::new::<B>(device);
        let config = bdh_model_config {
            n_layer: dims.n_layer as i32, n_embd: dims.n_embd as i32, n_head: dims.n_head as i32,
            latent: dims.latent as i32, vocab: dims.vocab as i32, rotary: dims.rotary as i32,
            rope_theta: dims.rope_theta, relu_threshold: dims.relu_threshold,
            alibi_slopes_host: alibi_slopes.map_or(std::ptr::null(), |s| s.as_ptr()),
        };
        let weights = bdh_model_weights {
            embed: B::device_ptr(&embed), encoder: B::device_ptr(&encoder), encoder_v: B::device_ptr(&encoder_v),
            decoder: B::device_ptr(&decoder), lm_head: B::device_ptr(&lm_head),
        };
        let mut raw = std::ptr::null_mut();
        ctx.check(unsafe { bdh_model_create(ctx.raw, &config, &weights, &mut raw) });
        Model { raw, ctx, dims, _embed: embed, _encoder: encoder, _encoder_v: encoder_v, _decoder: decoder,
            _lm_head: lm_head }
    }

    /// src/model/bdh.rs:254-256
    pub fn init_state(&self) -> ModelState<B> {
        ModelState::new(self.dims.n_layer)
    }

    /// Drop-in for BDH::forward_with_state (src/model/bdh.rs:309-313): the reference's signature.  Every layer's
    /// state is taken out of its LayerState (zeros on first use or on a shape change, :274-284), handed to the
    /// library as one pointer per layer (bdh_model_forward_layers: no copy into one allocation) and put back (:304);
    /// `state.position` advances by T (:445).
    pub fn forward_with_state(&self, tokens: Tensor<B, 2, Int>, state: &mut ModelState<B>) -> Tensor<B, 3> {
        assert_eq!(state.layers.len(), self.dims.n_layer, "model state layers mismatch"); // :314-318
        let [b, t] = tokens.dims();
        let (h, d, n) = (self.dims.n_head, self.dims.n_embd, self.dims.latent);
        let nq = if self.dims.rotary == RotaryEmbedding::Pope { 2 * n } else { n };
        let device = tokens.device();
        let rhos: Vec<Tensor<B, 4>> = state.layers.iter_mut().map(|layer| match layer.rho.take() {
            Some(r) if r.dims() == [b, h, nq, d] => r,
            _ => Tensor::<B, 4>::zeros([b, h, nq, d], &device),
        }).collect();
        let ptrs: Vec<*mut c_void> = rhos.iter().map(|r| B::device_ptr(r) as *mut c_void).collect();
        let logits = Tensor::<B, 3>::empty([b, t, self.dims.vocab], &device);
        self.ctx.check(unsafe {
            bdh_model_forward_layers(self.raw, B::int_device_ptr(&tokens), b as i32, t as i32, ptrs.as_ptr(), BDH_F32,
                std::ptr::null(), state.position as i64, std::ptr::null(), B::device_ptr(&logits),
                std::ptr::null_mut(), std::ptr::null_mut())
        });
        for (layer, rho) in state.layers.iter_mut().zip(rhos) {
            layer.rho = Some(rho);
        }
        state.position = state.position.saturating_add(t); // :445
        logits
    }
}

/// The pending state updates of a decode loop with deferred updates: one log per layer, for a batch of `batch`
/// sequences.  Owned by the caller next to the ModelState it belongs to; `Model::flush_deferred` (or the
/// `capacity`-th step by itself) applies what is pending.  No counterpart in the reference.
pub struct ModelLogs {
    raw: *mut bdh_model_logs,
    model: *mut bdh_model,
    batch: usize,
}

impl ModelLogs {
    pub fn pending(&self) -> usize {
        unsafe { bdh_model_logs_pending(self.raw) as usize }
    }
}

impl Drop for ModelLogs {
    fn drop(&mut self) {
        unsafe { bdh_model_logs_destroy(self.model, self.raw) };
    }
}

impl<B: HipPointers> Model<B> {
    /// Logs for decoding `batch` sequences with the state updates deferred, flushed every `capacity` tokens
    /// (RoPE models with n_embd 256 or 512; capacity 1..128 with capacity * n_embd <= 32768).  The logs must not
    /// outlive the model.
    pub fn deferred_logs(&self, batch: usize, capacity: usize) -> ModelLogs {
        let mut raw = std::ptr::null_mut();
        self.ctx.check(unsafe { bdh_model_logs_create(self.raw, batch as i32, BDH_F32, capacity as i32, &mut raw) });
        ModelLogs { raw, model: self.raw, batch }
    }

    /// One decode step (tokens [B,1]) of forward_with_state with the rank-1 updates of src/model/bdh.rs:298 logged
    /// instead of written: the layers' state tensors are read, not modified, until the logs are flushed.  Logits agree
    /// with forward_with_state to f32 rounding.  Call `flush_deferred` before anything else reads the state tensors.
    pub fn decode_step_deferred(&self, tokens: Tensor<B, 2, Int>, state: &mut ModelState<B>, logs: &mut ModelLogs)
        -> Tensor<B, 3> {
        let [b, t] = tokens.dims();
        assert_eq!(t, 1, "a deferred step takes one token per sequence");
        assert_eq!(b, logs.batch, "the logs were made for another batch size");
        let device = tokens.device();
        let ptrs: Vec<*mut c_void> = state.layers.iter().map(|layer| {
            let rho = layer.rho.as_ref().expect("a deferred step continues a state that a prompt call has made");
            B::device_ptr(rho) as *mut c_void
        }).collect();
        let logits = Tensor::<B, 3>::empty([b, 1, self.dims.vocab], &device);
        self.ctx.check(unsafe {
            bdh_model_forward_deferred_layers(self.raw, logs.raw, B::int_device_ptr(&tokens), b as i32, ptrs.as_ptr(),
                BDH_F32, state.position as i64, std::ptr::null(), B::device_ptr(&logits), std::ptr::null_mut())
        });
        state.position = state.position.saturating_add(1);
        logits
    }

    /// Applies the pending updates: afterwards the state tensors hold what forward_with_state would have left.
    pub fn flush_deferred(&self, state: &mut ModelState<B>, logs: &mut ModelLogs) {
        if logs.pending() == 0 {
            return;
        }
        let ptrs: Vec<*mut c_void> = state.layers.iter().map(|layer| {
            B::device_ptr(layer.rho.as_ref().expect("pending updates belong to a state")) as *mut c_void
        }).collect();
        self.ctx.check(unsafe { bdh_model_flush_layers(self.raw, logs.raw, ptrs.as_ptr()) });
    }
}

impl<B: HipPointers> Drop for Model<B> {
    fn drop(&mut self) {
        unsafe { bdh_model_destroy(self.raw) };
    }
}
