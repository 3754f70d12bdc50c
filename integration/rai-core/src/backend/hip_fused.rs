//! Safe wrappers over the fused launchers and the decoder drivers of librai_hip.so, for callers on the `Hip`
//! device that want more than one primitive per launch.
//!
//! They have no `impl Eval` of their own: rai's graph only ever holds primitives (rai-nn's `Linear`, `LayerNorm`,
//! `RmsNorm`, the rotary embedding and the attention blocks of rai-models are compositions), so these are what a
//! composition-matching pass in `eval()` calls once it has recognised such a group of nodes -- the C++ evaluator
//! of this library (`include/rai_graph.h`) does exactly that -- or what an application calls directly.
//!   linear       rai-nn/src/linear.rs:59-69 (+ hlops/activations.rs, residual add)
//!   layer_norm   rai-nn/src/layer_norm.rs:32-42
//!   rms_norm     rai-nn/src/rms_norm.rs:18-22, rai-models/src/llm/gemma.rs:42-54 (add_one)
//!   rope         rai-models/src/llm/phi2.rs:66-77, qwen2.rs:60-71
//!   attention    rai-models/src/llm/phi2.rs:244-262 (f32 scores), qwen2.rs:205-216
//!   sample_argmax examples/phi2/src/main.rs:29-50
//!   Decoder      rai-models/src/llm/{phi2,qwen2,gemma,phi3}.rs `Model::{new, fwd, clear_kv_cache}` and the greedy
//!                loop of examples/phi2/src/main.rs:72-95
use super::hip::HipData;
use super::hip_sys::*;
use std::ffi::{c_int, CString};

fn opt(t: Option<&HipData>) -> *const RaiHipTensor {
    t.map_or(std::ptr::null(), |d| d.desc() as *const _)
}

/// `act(x @ w^T + bias) + residual` into `out`; `act` is one of the `RAI_UN_*` activations or -1.
pub fn linear(dev: c_int, x: &HipData, w: &HipData, bias: Option<&HipData>, act: i32, residual: Option<&HipData>, out: &HipData) {
    check(unsafe { rai_hip_linear(dev, x.desc(), w.desc(), opt(bias), act, opt(residual), out.desc()) });
}

/// Several Linears over one input as one contraction (see `rai_hip_linear_packed` in the header).
#[allow(clippy::too_many_arguments)]
pub fn linear_packed(dev: c_int, x: &HipData, w: &HipData, bias: Option<&HipData>, bias2: Option<&HipData>, act: i32,
                     act_from: i32, residual: Option<&HipData>, glu: bool, k_splits: i32, out1: &HipData,
                     out2: Option<&HipData>) {
    check(unsafe {
        rai_hip_linear_packed(dev, x.desc(), w.desc(), opt(bias), opt(bias2), act, act_from, opt(residual), glu as i32,
                              k_splits, out1.desc(), opt(out2))
    });
}

pub fn layer_norm(dev: c_int, x: &HipData, w: Option<&HipData>, b: Option<&HipData>, eps: f64, out: &HipData) {
    check(unsafe { rai_hip_layer_norm(dev, x.desc(), opt(w), opt(b), eps, out.desc()) });
}

pub fn rms_norm(dev: c_int, x: &HipData, w: &HipData, eps: f64, add_one: bool, out: &HipData) {
    check(unsafe { rai_hip_rms_norm(dev, x.desc(), w.desc(), eps, add_one as i32, out.desc()) });
}

pub fn rope_tables(dev: c_int, theta: f64, rot_dim: i32, f64_powf: bool, cos: &HipData, sin: &HipData) {
    check(unsafe { rai_hip_rope_tables(dev, theta, rot_dim, f64_powf as i32, cos.desc(), sin.desc()) });
}

pub fn rope(dev: c_int, x: &HipData, cos: &HipData, sin: &HipData, rot_dim: i32, offset: i64, out: &HipData) {
    check(unsafe { rai_hip_rope(dev, x.desc(), cos.desc(), sin.desc(), rot_dim, offset, out.desc()) });
}

#[allow(clippy::too_many_arguments)]
pub fn attention(dev: c_int, q: &HipData, k: &HipData, v: &HipData, scale: f64, causal: bool, f32_scores: bool, out: &HipData) {
    check(unsafe { rai_hip_attention(dev, q.desc(), k.desc(), v.desc(), scale, causal as i32, f32_scores as i32, out.desc()) });
}

/// `apply_repeat_penalty` + `sample_argmax` of the example binaries on a `[rows, vocab]` logits tensor.
pub fn sample_argmax(dev: c_int, logits: &HipData, context: Option<&HipData>, repeat_penalty: f32, out: &HipData) {
    check(unsafe { rai_hip_sample_argmax(dev, logits.desc(), opt(context), repeat_penalty, out.desc()) });
}

/// `rai_hip_argmax` for code that may not allocate (HIP graph capture, serving loops): partial results live in a
/// fixed device array, at most 65536 rows, calls on one GPU must not overlap.
pub fn argmax_static(dev: c_int, x: &HipData, dim: i32, keep_dim: bool, out: &HipData) {
    check(unsafe { rai_hip_argmax_static(dev, x.desc(), dim, keep_dim as i32, out.desc()) });
}

pub fn sync(dev: c_int) {
    check(unsafe { rai_hip_sync(dev) });
}

/// (bytes in use, bytes pooled, device allocations made) of the library's allocator on `dev`.
pub fn mem_stats(dev: c_int) -> (u64, u64, u64) {
    let (mut a, mut b, mut n) = (0u64, 0u64, 0u64);
    check(unsafe { rai_hip_mem_stats(dev, &mut a, &mut b, &mut n) });
    (a, b, n)
}

pub fn trim(dev: c_int) {
    check(unsafe { rai_hip_trim(dev) });
}

/// A whole decoder-only model resident on the GPU, parameters addressed by the names `Module::named_params`
/// yields (rai-core/src/nn.rs:183-205; renames at rai-models/src/llm/phi2.rs:307-313).
pub struct Decoder {
    h: *mut RaiHipDecoder,
    vocab: usize,
}

impl Decoder {
    pub fn create(dev: c_int, cfg: &RaiHipDecoderConfig) -> Self {
        let mut h = std::ptr::null_mut();
        check(unsafe { rai_hip_init(dev) });
        check(unsafe { rai_hip_decoder_create(dev, cfg, &mut h) });
        Self { h, vocab: cfg.vocab_size as usize }
    }

    /// `(name, element count)` of every parameter the driver expects.
    pub fn param_names(&self) -> Vec<(String, i64)> {
        let mut n = 0i32;
        check(unsafe { rai_hip_decoder_param_count(self.h, &mut n) });
        (0..n)
            .map(|i| {
                let mut buf = vec![0u8; 256];
                let mut numel = 0i64;
                check(unsafe { rai_hip_decoder_param_name(self.h, i, buf.as_mut_ptr() as *mut _, buf.len(), &mut numel) });
                let end = buf.iter().position(|&c| c == 0).unwrap_or(buf.len());
                (String::from_utf8_lossy(&buf[..end]).into_owned(), numel)
            })
            .collect()
    }

    /// `[rows, cols]` of parameter `i` (a vector has one row).
    pub fn param_shape(&self, i: i32) -> (i64, i64) {
        let (mut r, mut c) = (0i64, 0i64);
        check(unsafe { rai_hip_decoder_param_shape(self.h, i, &mut r, &mut c) });
        (r, c)
    }

    /// One parameter from host bytes in the model dtype's storage form, e.g. in a loop over
    /// `model.named_params()` with `safetensors::View::data(&tensor)`.
    pub fn load_param(&self, name: &str, bytes: &[u8]) {
        let c = CString::new(name).unwrap();
        check(unsafe { rai_hip_decoder_load_param(self.h, c.as_ptr(), bytes.as_ptr() as *const _, bytes.len()) });
    }

    /// `Module::update_by_safetensors` (rai-core/src/nn.rs:39-55) from local files.
    pub fn load_safetensors(&self, paths: &[&str]) {
        let owned: Vec<CString> = paths.iter().map(|p| CString::new(*p).unwrap()).collect();
        let ptrs: Vec<*const _> = owned.iter().map(|c| c.as_ptr()).collect();
        check(unsafe { rai_hip_decoder_load_safetensors(self.h, ptrs.as_ptr(), ptrs.len() as i32) });
    }

    /// `Model::fwd`: ids `[batch, seq]` appended after the cached context; last-position logits `[batch, vocab]`
    /// and the greedy token per sequence.
    pub fn forward(&self, ids: &[u32], batch: usize, seq: usize) -> (Vec<f32>, Vec<u32>) {
        assert_eq!(ids.len(), batch * seq);
        let mut logits = vec![0f32; batch * self.vocab];
        let mut toks = vec![0u32; batch];
        check(unsafe {
            rai_hip_decoder_forward(self.h, ids.as_ptr(), batch as i32, seq as i32, logits.as_mut_ptr(), toks.as_mut_ptr())
        });
        (logits, toks)
    }

    /// The layer stack with both ends open: `rows` (`[batch * seq, hidden]` in the model dtype's storage form, as raw
    /// bytes) stand in for the embedding lookup; returns the residual stream after the last layer as f32, before the
    /// final norm.  With a one-layer model that is what `DecoderLayer::fwd` returns.
    pub fn forward_hidden(&self, rows: &[u8], batch: usize, seq: usize, hidden: usize) -> Vec<f32> {
        let mut out = vec![0f32; batch * seq * hidden];
        check(unsafe {
            rai_hip_decoder_forward_hidden(self.h, std::ptr::null(), rows.as_ptr() as *const std::ffi::c_void, batch as i32,
                                           seq as i32, out.as_mut_ptr(), std::ptr::null_mut(), std::ptr::null_mut())
        });
        out
    }

    /// Greedy decode on the device: `[batch, n_new]` tokens, prefill and decode milliseconds.
    pub fn generate(&self, prompt: &[u32], batch: usize, prompt_len: usize, n_new: usize) -> (Vec<u32>, f32, f32) {
        let mut toks = vec![0u32; batch * n_new];
        let (mut pre, mut dec) = (0f32, 0f32);
        check(unsafe {
            rai_hip_decoder_generate(self.h, prompt.as_ptr(), batch as i32, prompt_len as i32, n_new as i32, toks.as_mut_ptr(),
                                     &mut pre, &mut dec)
        });
        (toks, pre, dec)
    }

    /// The example binaries' loop: repeat penalty over the last `repeat_last_n` tokens, last-maximum argmax, stop
    /// after `eos_token`.  Returns the tokens and how many each sequence generated.
    #[allow(clippy::too_many_arguments)]
    pub fn generate_sampled(&self, prompt: &[u32], batch: usize, prompt_len: usize, n_new: usize, repeat_penalty: f32,
                            repeat_last_n: usize, eos_token: Option<u32>) -> (Vec<u32>, Vec<i32>) {
        let mut toks = vec![0u32; batch * n_new];
        let mut n_gen = vec![0i32; batch];
        let (mut pre, mut dec) = (0f32, 0f32);
        check(unsafe {
            rai_hip_decoder_generate_sampled(self.h, prompt.as_ptr(), batch as i32, prompt_len as i32, n_new as i32,
                                             repeat_penalty, repeat_last_n as i32, eos_token.map_or(-1, |t| t as i64),
                                             toks.as_mut_ptr(), n_gen.as_mut_ptr(), &mut pre, &mut dec)
        });
        (toks, n_gen)
    }

    pub fn clear_kv_cache(&self) {
        check(unsafe { rai_hip_decoder_clear_kv_cache(self.h) });
    }

    pub fn context_len(&self) -> usize {
        let mut n = 0i32;
        check(unsafe { rai_hip_decoder_context_len(self.h, &mut n) });
        n as usize
    }

    pub fn dtype(&self) -> i32 {
        let mut dt = 0i32;
        check(unsafe { rai_hip_decoder_dtype(self.h, &mut dt) });
        dt
    }
}

impl Drop for Decoder {
    fn drop(&mut self) {
        unsafe { rai_hip_decoder_destroy(self.h) };
    }
}

/// The shard files a `model.safetensors.index.json` names (rai/src/lib.rs:17-42 without the hub download).
pub fn safetensors_index_files(index_json: &str) -> Vec<String> {
    let c = CString::new(index_json).unwrap();
    let mut buf = vec![0u8; 1 << 16];
    let mut n = 0i32;
    check(unsafe { rai_hip_safetensors_index_files(c.as_ptr(), buf.as_mut_ptr() as *mut _, buf.len(), &mut n) });
    let end = buf.iter().position(|&c| c == 0).unwrap_or(buf.len());
    let s = String::from_utf8_lossy(&buf[..end]).into_owned();
    if n == 0 { vec![] } else { s.split('\n').map(str::to_owned).collect() }
}
