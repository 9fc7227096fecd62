//! LlamaModel on the GPU: the replacement for `LlamaModel::forward` (src/models/llama.rs:181-206) and for the
//! per-token loop of `src/main.rs:340-378`, over the C ABI in `ffi.rs`.
//!
//! UNCOMPILED: written where no Rust toolchain exists; it uses only what the reference crate exports
//! (`Tensor::data_ref`, `Tensor::from_array_no_grad`, `LlamaModel::{config, named_parameters}`).
//!
//! Use: build the CPU model and load its weights as today, then
//!     let gpu = GpuLlama::from_model(&model);          // uploads every parameter once
//!     let logits = gpu.forward(input_ids);             // same [1, S, V] tensor as LlamaModel::forward
//!     let ids = gpu.decode_greedy(first_id, 128);      // 128 tokens without leaving the GPU
use crate::autograd::Tensor;
use crate::ffi;
use crate::models::llama::LlamaModel;
use std::ffi::CString;
use std::os::raw::{c_int, c_void};

pub struct GpuLlama {
    ctx: *mut ffi::lumen_ctx,
    model: *mut ffi::lumen_llama,
    vocab: usize,
}

impl GpuLlama {
    /// LlamaModel::new + ModelLoader::load_llama_weights, device side: one `lumen_llama_set_param` per entry of
    /// `named_parameters()` (src/models/llama.rs:218-279; same Hugging Face names).
    pub fn from_model(cpu: &LlamaModel) -> Self {
        let c = &cpu.config;
        let cfg = ffi::lumen_llama_config {
            vocab_size: c.vocab_size as c_int,
            hidden_size: c.hidden_size as c_int,
            intermediate_size: c.intermediate_size as c_int,
            num_hidden_layers: c.num_hidden_layers as c_int,
            num_attention_heads: c.num_attention_heads as c_int,
            num_key_value_heads: c.num_key_value_heads as c_int,
            rms_norm_eps: c.rms_norm_eps,
            max_seq_len: c.max_seq_len as c_int,
            rope_theta: c.rope_theta,
            head_dim: 0,
            qk_norm: 0,
            tie_embeddings: 0,
            weight_dtype: ffi::LUMEN_DTYPE_F32,
        };
        let mut ctx = std::ptr::null_mut();
        let mut model = std::ptr::null_mut();
        unsafe {
            ffi::check(ffi::lumen_ctx_create(0, &mut ctx));
            ffi::check(ffi::lumen_llama_create(ctx, &cfg, &mut model));
        }
        for (name, t) in cpu.named_parameters() {
            let data = t.data_ref();
            let shape: Vec<i64> = data.shape().iter().map(|&d| d as i64).collect();
            let host = data.as_standard_layout();
            let cname = CString::new(name).unwrap();
            unsafe {
                ffi::check(ffi::lumen_llama_set_param(
                    model,
                    cname.as_ptr(),
                    host.as_ptr() as *const c_void,
                    ffi::LUMEN_DTYPE_F32,
                    shape.as_ptr(),
                    shape.len() as c_int,
                ));
            }
        }
        GpuLlama { ctx, model, vocab: c.vocab_size }
    }

    /// LlamaModel::forward: ids [1, S] as f32 in, logits [1, S, V] out.  The KV caches live in the handle, so the
    /// `caches` / `_pos` arguments of the reference signature have nothing to carry here.
    pub fn forward(&self, input_ids: Tensor) -> Tensor {
        let ids: Vec<f32> = input_ids.data_ref().iter().copied().collect();
        let s = ids.len();
        let mut logits = vec![0f32; s * self.vocab];
        unsafe { ffi::check(ffi::lumen_llama_forward(self.model, ids.as_ptr(), s as c_int, logits.as_mut_ptr(), 1)) };
        Tensor::from_array_no_grad(ndarray::Array::from_shape_vec((1, s, self.vocab), logits).unwrap().into_dyn())
    }

    /// Logits of the last position only: what `main.rs:155-163` keeps of a prompt pass.
    pub fn forward_last(&self, ids: &[f32]) -> Vec<f32> {
        let mut logits = vec![0f32; self.vocab];
        unsafe { ffi::check(ffi::lumen_llama_forward(self.model, ids.as_ptr(), ids.len() as c_int, logits.as_mut_ptr(), 0)) };
        logits
    }

    /// `n` greedy tokens after `first_id` (the loop of main.rs:340-378 with arg-max in place of sample_top_p).
    pub fn decode_greedy(&self, first_id: usize, n: usize) -> Vec<i32> {
        let mut out = vec![0i32; n];
        unsafe {
            ffi::check(ffi::lumen_llama_decode_greedy(self.model, first_id as c_int, n as c_int, out.as_mut_ptr(), std::ptr::null_mut()))
        };
        out
    }

    /// reset_kv_caches (src/models/llama.rs:172-176)
    pub fn reset_kv_caches(&self) {
        unsafe { ffi::check(ffi::lumen_llama_reset(self.model)) };
    }
}

impl Drop for GpuLlama {
    fn drop(&mut self) {
        unsafe {
            ffi::lumen_llama_destroy(self.model);
            ffi::lumen_ctx_destroy(self.ctx);
        }
    }
}
