//! The safe layer a metallic-foundry maintainer adds on top of the raw declarations of lib.rs: the error mapping, the
//! TensorArg conversion and the bodies of the two compiled steps. Source text only - this file names types of
//! crates/metallic-foundry (TensorArg, MetalError, Dtype, Foundry, FastBindings ...) and therefore compiles inside that
//! crate, not inside foundry_attn_sys; copy it to crates/metallic-foundry/src/hip/attn.rs and add
//! `foundry_attn_sys = { path = ... }` to that crate's dependencies. It was not compiled in the image this library is
//! built in (no rustc there); the same calls, in the same order, are exercised by the C++ mirror
//! (test-burn_amd/host/foundry.hpp, tests/host/host_test.cpp).
use std::ffi::CStr;
use std::os::raw::c_int;

use foundry_attn_sys::*;

use crate::error::MetalError; // src/error.rs:22-75
use crate::types::TensorArg; // src/types/mod.rs:339-347
use metallic_sdk::tensor::Dtype; // crates/metallic-sdk/src/tensor.rs:7-30 (fa_dtype keeps its discriminants)

/// fa_status -> Result<(), MetalError>, variant for variant.
pub fn check(status: fa_status) -> Result<(), MetalError> {
    if status == FA_OK {
        return Ok(());
    }
    let msg = unsafe { CStr::from_ptr(fa_last_error_string()) }.to_string_lossy().into_owned();
    Err(match status {
        FA_ERR_DEVICE_NOT_FOUND => MetalError::DeviceNotFound,
        FA_ERR_NULL_POINTER => MetalError::NullPointer,
        FA_ERR_INVALID_SHAPE => MetalError::InvalidShape(msg),
        FA_ERR_OUT_OF_MEMORY => MetalError::OutOfMemory,
        FA_ERR_OPERATION_NOT_SUPPORTED => MetalError::OperationNotSupported(msg), // bad head_dim / layout / kv_head_major=false
        FA_ERR_INVALID_OPERATION => MetalError::InvalidOperation(msg),
        FA_ERR_UNSUPPORTED_DTYPE => MetalError::UnsupportedDtype {
            operation: "foundry_attn",
            // the dtype the library refused, not a constant
            dtype: Dtype::from_discriminant(unsafe { fa_last_error_dtype() }).unwrap_or(Dtype::F16),
        },
        FA_ERR_INPUT_NOT_FOUND => MetalError::InputNotFound(msg), // a TensorArg without a buffer
        _ => MetalError::OperationFailed(msg),                    // HIP runtime failures, a polled merge that gave up
    })
}

/// TensorArg -> fa_tensor_arg: the buffer's HIP device pointer, byte offset, dtype discriminant, dims, element strides.
pub fn arg(t: &TensorArg) -> fa_tensor_arg {
    let mut a = fa_tensor_arg {
        buffer: t.buffer.as_ref().map_or(std::ptr::null_mut(), |b| b.device_ptr()),
        offset: t.offset,
        dtype: t.dtype as u32,
        rank: t.dims.len() as u32,
        dims: [0; 4],
        strides: [0; 4],
    };
    for (i, d) in t.dims.iter().take(4).enumerate() {
        a.dims[i] = *d;
    }
    for (i, s) in t.strides.iter().take(4).enumerate() {
        a.strides[i] = *s;
    }
    a
}

/// An absent optional tensor (gamma, biases, Q8_0 scales, q_rot): a null buffer.
pub fn opt(t: Option<&TensorArg>) -> fa_tensor_arg {
    match t {
        Some(t) => arg(t),
        None => fa_tensor_arg { buffer: std::ptr::null_mut(), offset: 0, dtype: FA_DTYPE_F16, rank: 0, dims: [0; 4], strides: [0; 4] },
    }
}

// CompiledKvPrepFusedStep::execute (src/metals/kv_prep/step.rs:92-130), the body after
// `let params = self.step.params.resolve(bindings);` - in place of `foundry.run(&kernel)`.
pub fn kv_prep_fused_execute(
    ctx: *mut fa_ctx,
    q: &TensorArg, k: &TensorArg, v: &TensorArg, q_rot: &TensorArg, k_cache: &TensorArg, v_cache: &TensorArg,
    cos: &TensorArg, sin: &TensorArg,
    p: &crate::metals::kv_prep::KvPrepFusedParamsResolved, // src/metals/kv_prep/mod.rs:79-114: the same 13 fields, same order
) -> Result<(), MetalError> {
    let params = fa_kv_prep_fused_params {
        d_model: p.d_model, kv_dim: p.kv_dim, head_dim: p.head_dim, n_heads: p.n_heads, n_kv_heads: p.n_kv_heads,
        group_size: p.group_size, seq_len: p.seq_len, position_offset: p.position_offset, max_seq_len: p.max_seq_len,
        total_elements: p.total_elements, rope_mode: p.rope_mode, layer_idx: p.layer_idx,
        no_rope_layer_step: p.no_rope_layer_step,
    };
    check(unsafe {
        fa_kv_prep_fused(ctx, &arg(q), &arg(k), &arg(v), &arg(q_rot), &arg(k_cache), &arg(v_cache), &arg(cos), &arg(sin), &params)
    })
}

// CompiledFlashAttentionStep::execute (src/metals/sdpa/step.rs:160-503): everything after the resolution of the
// DynamicValue fields collapses to one call; the routing (m == 1 -> decode, m > 1 -> prefill), the stride and layout
// inference (src/metals/flashattention/step.rs:668-756, 797-831, 1000-1042), the kv_head_major check (:193-197) and
// scale = 1/sqrt(head_dim) live behind it.
#[allow(clippy::too_many_arguments)]
pub fn flash_attention_execute(
    ctx: *mut fa_ctx,
    q: &TensorArg, k: &TensorArg, v: &TensorArg, output: &TensorArg,
    causal: bool, query_offset: u32, n_heads: u32, head_dim: u32, kv_seq_len: u32, m: u32, kv_head_major: bool,
) -> Result<(), MetalError> {
    check(unsafe {
        fa_flash_attention(ctx, &arg(q), &arg(k), &arg(v), &arg(output), causal as c_int, query_offset, n_heads, head_dim,
                           kv_seq_len, m, kv_head_major as c_int)
    })
}

// A decode step (m == 1) of one layer as ONE launch instead of the KvPrepFused + FlashAttention pair
// (models/llama.json:529-565): raw projections in, token appended and attended. `d_position` is a device u32 that a
// captured graph replays against (fa_u32_add advances it once per step); null = params.position_offset.
#[allow(clippy::too_many_arguments)]
pub fn decode_step_fused_execute(
    ctx: *mut fa_ctx,
    q: &TensorArg, k: &TensorArg, v: &TensorArg, q_rot: Option<&TensorArg>, k_cache: &TensorArg, v_cache: &TensorArg,
    cos: &TensorArg, sin: &TensorArg, output: &TensorArg, params: &fa_kv_prep_fused_params, d_position: *const u32,
    kv_len_bound: u32,
) -> Result<(), MetalError> {
    check(unsafe {
        fa_decode_step_fused(ctx, &arg(q), &arg(k), &arg(v), &opt(q_rot), &arg(k_cache), &arg(v_cache), &arg(cos), &arg(sin),
                             &arg(output), params, d_position, kv_len_bound)
    })
}

// Foundry gains one field, `hip_ctx: *mut fa_ctx`: fa_ctx_create in Foundry::new (src/lib.rs:57-61), fa_ctx_destroy in
// Drop, fa_synchronize in Foundry::synchronize (src/lib.rs:175-188), fa_start_capture / fa_end_capture / fa_graph_launch
// for start_capture / end_capture (src/lib.rs:94-164). One context per Foundry (it is used through &mut,
// src/lib.rs:44-53). A process that drives several contexts or streams on one GPU at the same time sets
// FOUNDRY_ATTN_DECODE_MERGE=1 (see fa_set_decode_variant in the header).
