//! Raw FFI declarations of libfoundry_attn.so: the KV-cache attention path of metallic-foundry (KvPrepFused,
//! FlashAttention and the ops either side of them) on AMD MI355X. GENERATED from include/foundry_attn.h by
//! ffi/foundry_attn_sys/generate.py - edit the header, not this file. The header's comments name, for every entry
//! point, the interface of crates/metallic-foundry it stands in for.
#![allow(non_camel_case_types, non_upper_case_globals)]
use std::os::raw::{c_char, c_int, c_void};

/// 0 = ok; the other values are the variants of MetalError this path raises (src/error.rs:22-75).
pub type fa_status = i32;

pub const FA_OK: fa_status = 0;
pub const FA_ERR_DEVICE_NOT_FOUND: fa_status = 1;
pub const FA_ERR_NULL_POINTER: fa_status = 2;
pub const FA_ERR_INVALID_SHAPE: fa_status = 3;
pub const FA_ERR_OUT_OF_MEMORY: fa_status = 4;
pub const FA_ERR_OPERATION_NOT_SUPPORTED: fa_status = 5;
pub const FA_ERR_INVALID_OPERATION: fa_status = 6;
pub const FA_ERR_UNSUPPORTED_DTYPE: fa_status = 7;
pub const FA_ERR_OPERATION_FAILED: fa_status = 8;
pub const FA_ERR_INPUT_NOT_FOUND: fa_status = 9;

pub type fa_dtype = u32;
pub const FA_DTYPE_F32: fa_dtype = 0;
pub const FA_DTYPE_F16: fa_dtype = 1;
pub const FA_DTYPE_BF16: fa_dtype = 2;
pub const FA_DTYPE_Q4_0: fa_dtype = 3;
pub const FA_DTYPE_Q8_0: fa_dtype = 7;
pub const FA_DTYPE_I8: fa_dtype = 15;
pub const FA_DTYPE_I16: fa_dtype = 16;
pub const FA_DTYPE_I32: fa_dtype = 17;
pub const FA_DTYPE_U8: fa_dtype = 18;
pub const FA_DTYPE_U16: fa_dtype = 19;
pub const FA_DTYPE_U32: fa_dtype = 20;
pub const FA_DTYPE_F64: fa_dtype = 21;

pub type fa_weight_layout = u32;
pub const FA_WEIGHT_LAYOUT_ROW_MAJOR: fa_weight_layout = 0;
pub const FA_WEIGHT_LAYOUT_CANONICAL: fa_weight_layout = 1;

pub const FA_ROPE_MODE_NEOX: u32 = 0;
pub const FA_ROPE_MODE_NORMAL: u32 = 1;
pub const FA_SAGE_BLOCK: u32 = 32;

#[repr(C)]
pub struct fa_ctx {
    _private: [u8; 0],
}

#[repr(C)]
pub struct fa_graph {
    _private: [u8; 0],
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fa_tensor_arg {
    pub buffer: *mut c_void,
    pub offset: usize,
    pub dtype: u32,
    pub rank: u32,
    pub dims: [usize; 4],
    pub strides: [usize; 4],
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fa_kv_prep_fused_params {
    pub d_model: u32,
    pub kv_dim: u32,
    pub head_dim: u32,
    pub n_heads: u32,
    pub n_kv_heads: u32,
    pub group_size: u32,
    pub seq_len: u32,
    pub position_offset: u32,
    pub max_seq_len: u32,
    pub total_elements: u32,
    pub rope_mode: u32,
    pub layer_idx: u32,
    pub no_rope_layer_step: u32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fa_decode_variant {
    pub keys_per_split: u32,
    pub merge: u32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fa_paged_kv {
    pub k_pool: *mut c_void,
    pub v_pool: *mut c_void,
    pub block_table: *const i32,
    pub seq_lens: *const u32,
    pub n_blocks: u32,
    pub n_kv_heads: u32,
    pub block_size: u32,
    pub head_dim: u32,
    pub n_seqs: u32,
    pub max_blocks_per_seq: u32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fa_fused_qkv_params {
    pub k_dim: u32,
    pub n_dim: u32,
    pub n_kv: u32,
    pub m: u32,
    pub weights_per_block: u32,
    pub layout: u32,
    pub epsilon: f32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fa_matmul_params {
    pub m: u32,
    pub n: u32,
    pub k: u32,
    pub transpose_a: u32,
    pub transpose_b: u32,
    pub alpha: f32,
    pub beta: f32,
    pub weights_per_block: u32,
    pub activation: u32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fa_sage_cache {
    pub k_q: *mut c_void,
    pub k_scale: *mut c_void,
    pub k_tail: *mut c_void,
    pub v: *mut c_void,
    pub q_q: *mut c_void,
    pub k_mean: *mut f32,
    pub q_scale: *mut f32,
    pub n_heads: u32,
    pub n_kv_heads: u32,
    pub capacity: u32,
    pub head_dim: u32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fa_rope_params {
    pub dim: u32,
    pub seq_len: u32,
    pub position_offset: u32,
    pub total_elements: u32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fa_kv_cache_write_params {
    pub n_kv_heads: u32,
    pub head_dim: u32,
    pub input_seq_len: u32,
    pub position_offset: u32,
    pub max_seq_len: u32,
    pub total_elements: u32,
    pub layer_idx: u32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fa_kv_cache_write_repeat_params {
    pub n_kv_heads: u32,
    pub n_heads: u32,
    pub group_size: u32,
    pub head_dim: u32,
    pub input_seq_len: u32,
    pub position_offset: u32,
    pub max_seq_len: u32,
    pub total_elements: u32,
    pub layer_idx: u32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fa_kv_cache_read_params {
    pub n_kv_heads: u32,
    pub head_dim: u32,
    pub seq_len: u32,
    pub max_seq_len: u32,
    pub total_elements: u32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fa_kv_rearrange_params {
    pub kv_dim: u32,
    pub row_stride: u32,
    pub kv_head_dim: u32,
    pub n_heads: u32,
    pub n_kv_heads: u32,
    pub head_dim: u32,
    pub seq: u32,
    pub total_elements: u32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fa_repeat_kv_heads_params {
    pub group_size: u32,
    pub batch: u32,
    pub n_kv_heads: u32,
    pub n_heads: u32,
    pub seq: u32,
    pub head_dim: u32,
    pub cache_stride: u32,
    pub total_elements: u32,
}

#[link(name = "foundry_attn")]
extern "C" {
    pub fn fa_status_name(s: fa_status) -> *const c_char;
    pub fn fa_last_error_string() -> *const c_char;
    pub fn fa_last_error_dtype() -> u32;
    pub fn fa_ctx_create(device: c_int, out: *mut *mut fa_ctx) -> fa_status;
    pub fn fa_ctx_destroy(ctx: *mut fa_ctx) -> fa_status;
    pub fn fa_synchronize(ctx: *mut fa_ctx) -> fa_status;
    pub fn fa_ctx_stream(ctx: *mut fa_ctx) -> *mut c_void;
    pub fn fa_ctx_reserve_workspace(ctx: *mut fa_ctx, bytes: usize) -> fa_status;
    pub fn fa_start_capture(ctx: *mut fa_ctx) -> fa_status;
    pub fn fa_end_capture(ctx: *mut fa_ctx, out: *mut *mut fa_graph) -> fa_status;
    pub fn fa_graph_launch(ctx: *mut fa_ctx, graph: *mut fa_graph) -> fa_status;
    pub fn fa_graph_destroy(graph: *mut fa_graph) -> fa_status;
    pub fn fa_is_capturing(ctx: *mut fa_ctx) -> c_int;
    pub fn fa_profile_enable(ctx: *mut fa_ctx, on: c_int) -> fa_status;
    pub fn fa_profile_reset(ctx: *mut fa_ctx) -> fa_status;
    pub fn fa_profile_query(
        ctx: *mut fa_ctx,
        kernel_prefix: *const c_char,
        launches: *mut u64,
        total_ms: *mut f64,
    ) -> fa_status;
    pub fn fa_profile_clock_buffer(ctx: *mut fa_ctx, d_buffer: *mut c_void, n_workgroups: u32) -> fa_status;
    pub fn fa_stream_timer_start(ctx: *mut fa_ctx) -> fa_status;
    pub fn fa_stream_timer_stop(ctx: *mut fa_ctx, elapsed_ms: *mut f32) -> fa_status;
    pub fn fa_compute_units(ctx: *mut fa_ctx, n: *mut u32) -> fa_status;
    pub fn fa_device_alloc(ctx: *mut fa_ctx, bytes: usize, out: *mut *mut c_void) -> fa_status;
    pub fn fa_device_free(ctx: *mut fa_ctx, ptr: *mut c_void) -> fa_status;
    pub fn fa_upload(
        ctx: *mut fa_ctx,
        dst: *mut c_void,
        dst_offset: usize,
        src_host: *const c_void,
        bytes: usize,
    ) -> fa_status;
    pub fn fa_download(
        ctx: *mut fa_ctx,
        dst_host: *mut c_void,
        src: *const c_void,
        src_offset: usize,
        bytes: usize,
    ) -> fa_status;
    pub fn fa_device_memset(ctx: *mut fa_ctx, dst: *mut c_void, value: c_int, bytes: usize) -> fa_status;
    pub fn fa_device_copy(
        ctx: *mut fa_ctx,
        dst: *mut c_void,
        dst_offset: usize,
        src: *const c_void,
        src_offset: usize,
        bytes: usize,
    ) -> fa_status;
    pub fn fa_u32_add(ctx: *mut fa_ctx, d_values: *mut u32, n: u32, delta: u32) -> fa_status;
    pub fn fa_rope_tables_f16(
        rope_base: f32,
        head_dim: u32,
        pos_begin: u32,
        pos_end: u32,
        freq_factors: *const f32,
        cos_out_host: *mut u16,
        sin_out_host: *mut u16,
    ) -> fa_status;
    pub fn fa_kv_prep_fused(
        ctx: *mut fa_ctx,
        q: *const fa_tensor_arg,
        k: *const fa_tensor_arg,
        v: *const fa_tensor_arg,
        q_rot: *const fa_tensor_arg,
        k_cache: *const fa_tensor_arg,
        v_cache: *const fa_tensor_arg,
        cos: *const fa_tensor_arg,
        sin: *const fa_tensor_arg,
        params: *const fa_kv_prep_fused_params,
    ) -> fa_status;
    pub fn fa_kv_prep_fused_dyn(
        ctx: *mut fa_ctx,
        q: *const fa_tensor_arg,
        k: *const fa_tensor_arg,
        v: *const fa_tensor_arg,
        q_rot: *const fa_tensor_arg,
        k_cache: *const fa_tensor_arg,
        v_cache: *const fa_tensor_arg,
        cos: *const fa_tensor_arg,
        sin: *const fa_tensor_arg,
        params: *const fa_kv_prep_fused_params,
        d_position_offset: *const u32,
    ) -> fa_status;
    pub fn fa_flash_attention(
        ctx: *mut fa_ctx,
        q: *const fa_tensor_arg,
        k: *const fa_tensor_arg,
        v: *const fa_tensor_arg,
        output: *const fa_tensor_arg,
        causal: c_int,
        query_offset: u32,
        n_heads: u32,
        head_dim: u32,
        kv_seq_len: u32,
        m: u32,
        kv_head_major: c_int,
    ) -> fa_status;
    pub fn fa_flash_decode_dyn(
        ctx: *mut fa_ctx,
        q: *const fa_tensor_arg,
        k: *const fa_tensor_arg,
        v: *const fa_tensor_arg,
        output: *const fa_tensor_arg,
        n_heads: u32,
        head_dim: u32,
        d_position: *const u32,
        kv_len_add: u32,
        kv_len_bound: u32,
    ) -> fa_status;
    pub fn fa_decode_step_fused(
        ctx: *mut fa_ctx,
        q: *const fa_tensor_arg,
        k: *const fa_tensor_arg,
        v: *const fa_tensor_arg,
        q_rot: *const fa_tensor_arg,
        k_cache: *const fa_tensor_arg,
        v_cache: *const fa_tensor_arg,
        cos: *const fa_tensor_arg,
        sin: *const fa_tensor_arg,
        output: *const fa_tensor_arg,
        params: *const fa_kv_prep_fused_params,
        d_position: *const u32,
        kv_len_bound: u32,
    ) -> fa_status;
    pub fn fa_decode_step_fused_noalloc(
        ctx: *mut fa_ctx,
        q: *const fa_tensor_arg,
        k: *const fa_tensor_arg,
        v: *const fa_tensor_arg,
        q_rot: *const fa_tensor_arg,
        k_cache: *const fa_tensor_arg,
        v_cache: *const fa_tensor_arg,
        cos: *const fa_tensor_arg,
        sin: *const fa_tensor_arg,
        output: *const fa_tensor_arg,
        params: *const fa_kv_prep_fused_params,
        d_position: *const u32,
        kv_len_bound: u32,
    ) -> fa_status;
    pub fn fa_noalloc_scratch_bytes() -> usize;
    pub fn fa_set_decode_variant(ctx: *mut fa_ctx, variant: *const fa_decode_variant) -> fa_status;
    pub fn fa_set_decode_poll_spin_us(ctx: *mut fa_ctx, spin_us: u32) -> fa_status;
    pub fn fa_set_prefill_split_k(ctx: *mut fa_ctx, split_k: u32) -> fa_status;
    pub fn fa_set_prefill_variant(ctx: *mut fa_ctx, variant: u32) -> fa_status;
    pub fn fa_kv_prep_fused_paged(
        ctx: *mut fa_ctx,
        q: *const fa_tensor_arg,
        k: *const fa_tensor_arg,
        v: *const fa_tensor_arg,
        q_rot: *const fa_tensor_arg,
        cache: *const fa_paged_kv,
        seq_index: u32,
        cos: *const fa_tensor_arg,
        sin: *const fa_tensor_arg,
        params: *const fa_kv_prep_fused_params,
    ) -> fa_status;
    pub fn fa_kv_prep_decode_paged(
        ctx: *mut fa_ctx,
        q: *const fa_tensor_arg,
        k: *const fa_tensor_arg,
        v: *const fa_tensor_arg,
        q_rot: *const fa_tensor_arg,
        cache: *const fa_paged_kv,
        cos: *const fa_tensor_arg,
        sin: *const fa_tensor_arg,
        params: *const fa_kv_prep_fused_params,
    ) -> fa_status;
    pub fn fa_flash_decode_paged(
        ctx: *mut fa_ctx,
        q: *const fa_tensor_arg,
        cache: *const fa_paged_kv,
        output: *const fa_tensor_arg,
        n_heads: u32,
        kv_len_add: u32,
        kv_len_bound: u32,
    ) -> fa_status;
    pub fn fa_decode_step_fused_paged(
        ctx: *mut fa_ctx,
        q: *const fa_tensor_arg,
        k: *const fa_tensor_arg,
        v: *const fa_tensor_arg,
        q_rot: *const fa_tensor_arg,
        cache: *const fa_paged_kv,
        cos: *const fa_tensor_arg,
        sin: *const fa_tensor_arg,
        output: *const fa_tensor_arg,
        params: *const fa_kv_prep_fused_params,
        kv_len_bound: u32,
    ) -> fa_status;
    pub fn fa_flash_prefill_paged(
        ctx: *mut fa_ctx,
        q: *const fa_tensor_arg,
        cache: *const fa_paged_kv,
        seq_index: u32,
        output: *const fa_tensor_arg,
        causal: c_int,
        query_offset: u32,
        n_heads: u32,
        kv_seq_len: u32,
        m: u32,
    ) -> fa_status;
    pub fn fa_paged_gather(
        ctx: *mut fa_ctx,
        cache: *const fa_paged_kv,
        seq_index: u32,
        seq_len: u32,
        k_out: *mut c_void,
        v_out: *mut c_void,
        out_capacity: u32,
    ) -> fa_status;
    pub fn fa_kv_prefix_copy(
        ctx: *mut fa_ctx,
        src: *const fa_tensor_arg,
        dst: *const fa_tensor_arg,
        prefix_len: usize,
    ) -> fa_status;
    pub fn fa_kv_prefix_copy_batch(
        ctx: *mut fa_ctx,
        src: *const fa_tensor_arg,
        dst: *const fa_tensor_arg,
        n: u32,
        prefix_len: usize,
    ) -> fa_status;
    pub fn fa_align_capacity(capacity: usize) -> usize;
    pub fn fa_grown_capacity(
        allocated: usize,
        required_len: usize,
        max_context_len: usize,
        growth_factor: f32,
    ) -> usize;
    pub fn fa_paged_copy_blocks(
        ctx: *mut fa_ctx,
        cache: *const fa_paged_kv,
        d_src_ids: *const i32,
        d_dst_ids: *const i32,
        n_pairs: u32,
    ) -> fa_status;
    pub fn fa_fused_qkv(
        ctx: *mut fa_ctx,
        w_q: *const fa_tensor_arg,
        s_q: *const fa_tensor_arg,
        w_k: *const fa_tensor_arg,
        s_k: *const fa_tensor_arg,
        w_v: *const fa_tensor_arg,
        s_v: *const fa_tensor_arg,
        input: *const fa_tensor_arg,
        out_q: *const fa_tensor_arg,
        out_k: *const fa_tensor_arg,
        out_v: *const fa_tensor_arg,
        bias_q: *const fa_tensor_arg,
        bias_k: *const fa_tensor_arg,
        bias_v: *const fa_tensor_arg,
        gamma: *const fa_tensor_arg,
        params: *const fa_fused_qkv_params,
    ) -> fa_status;
    pub fn fa_fused_qkv_kv_prep(
        ctx: *mut fa_ctx,
        w_q: *const fa_tensor_arg,
        s_q: *const fa_tensor_arg,
        w_k: *const fa_tensor_arg,
        s_k: *const fa_tensor_arg,
        w_v: *const fa_tensor_arg,
        s_v: *const fa_tensor_arg,
        input: *const fa_tensor_arg,
        bias_q: *const fa_tensor_arg,
        bias_k: *const fa_tensor_arg,
        bias_v: *const fa_tensor_arg,
        gamma: *const fa_tensor_arg,
        qkv_params: *const fa_fused_qkv_params,
        q_rot: *const fa_tensor_arg,
        k_cache: *const fa_tensor_arg,
        v_cache: *const fa_tensor_arg,
        cos: *const fa_tensor_arg,
        sin: *const fa_tensor_arg,
        params: *const fa_kv_prep_fused_params,
    ) -> fa_status;
    pub fn fa_fused_qkv_kv_prep_paged(
        ctx: *mut fa_ctx,
        w_q: *const fa_tensor_arg,
        s_q: *const fa_tensor_arg,
        w_k: *const fa_tensor_arg,
        s_k: *const fa_tensor_arg,
        w_v: *const fa_tensor_arg,
        s_v: *const fa_tensor_arg,
        input: *const fa_tensor_arg,
        bias_q: *const fa_tensor_arg,
        bias_k: *const fa_tensor_arg,
        bias_v: *const fa_tensor_arg,
        gamma: *const fa_tensor_arg,
        qkv_params: *const fa_fused_qkv_params,
        q_rot: *const fa_tensor_arg,
        cache: *const fa_paged_kv,
        seq_index: u32,
        cos: *const fa_tensor_arg,
        sin: *const fa_tensor_arg,
        params: *const fa_kv_prep_fused_params,
    ) -> fa_status;
    pub fn fa_matmul(
        ctx: *mut fa_ctx,
        a: *const fa_tensor_arg,
        b: *const fa_tensor_arg,
        b_scales: *const fa_tensor_arg,
        output: *const fa_tensor_arg,
        bias: *const fa_tensor_arg,
        c: *const fa_tensor_arg,
        params: *const fa_matmul_params,
    ) -> fa_status;
    pub fn fa_set_gemm_min_m(ctx: *mut fa_ctx, min_m: u32) -> fa_status;
    pub fn fa_set_gemm_variant(ctx: *mut fa_ctx, variant: u32) -> fa_status;
    pub fn fa_sage_k_mean(
        ctx: *mut fa_ctx,
        k: *const c_void,
        n_kv_heads: u32,
        capacity: u32,
        head_dim: u32,
        kv_len: u32,
        mean_out: *mut f32,
    ) -> fa_status;
    pub fn fa_sage_quantize_k(
        ctx: *mut fa_ctx,
        k: *const c_void,
        mean: *const f32,
        n_kv_heads: u32,
        capacity: u32,
        head_dim: u32,
        row_begin: u32,
        row_end: u32,
        k_q: *mut c_void,
        k_scale: *mut c_void,
    ) -> fa_status;
    pub fn fa_sage_quantize_q(
        ctx: *mut fa_ctx,
        q: *const c_void,
        n_heads: u32,
        head_dim: u32,
        q_q: *mut c_void,
        q_scale: *mut f32,
    ) -> fa_status;
    pub fn fa_sage_decode(
        ctx: *mut fa_ctx,
        q_q: *const c_void,
        q_scale: *const f32,
        k_q: *const c_void,
        k_scale: *const c_void,
        v: *const c_void,
        out: *mut c_void,
        n_heads: u32,
        n_kv_heads: u32,
        head_dim: u32,
        capacity: u32,
        kv_len: u32,
    ) -> fa_status;
    pub fn fa_sage_cache_build(
        ctx: *mut fa_ctx,
        k_f16: *const c_void,
        kv_len: u32,
        cache: *const fa_sage_cache,
    ) -> fa_status;
    pub fn fa_sage_decode_step(
        ctx: *mut fa_ctx,
        q: *const fa_tensor_arg,
        k: *const fa_tensor_arg,
        v: *const fa_tensor_arg,
        cache: *const fa_sage_cache,
        cos: *const fa_tensor_arg,
        sin: *const fa_tensor_arg,
        output: *const fa_tensor_arg,
        params: *const fa_kv_prep_fused_params,
        d_position: *const u32,
        kv_len_bound: u32,
    ) -> fa_status;
    pub fn fa_set_sage_step_variant(ctx: *mut fa_ctx, variant: u32) -> fa_status;
    pub fn fa_rope(
        ctx: *mut fa_ctx,
        input: *const fa_tensor_arg,
        output: *const fa_tensor_arg,
        cos: *const fa_tensor_arg,
        sin: *const fa_tensor_arg,
        params: *const fa_rope_params,
    ) -> fa_status;
    pub fn fa_kv_cache_write(
        ctx: *mut fa_ctx,
        input: *const fa_tensor_arg,
        cache: *const fa_tensor_arg,
        params: *const fa_kv_cache_write_params,
    ) -> fa_status;
    pub fn fa_kv_cache_write_repeat_kv_heads(
        ctx: *mut fa_ctx,
        input: *const fa_tensor_arg,
        cache: *const fa_tensor_arg,
        params: *const fa_kv_cache_write_repeat_params,
    ) -> fa_status;
    pub fn fa_kv_cache_read(
        ctx: *mut fa_ctx,
        cache: *const fa_tensor_arg,
        output: *const fa_tensor_arg,
        params: *const fa_kv_cache_read_params,
    ) -> fa_status;
    pub fn fa_kv_rearrange(
        ctx: *mut fa_ctx,
        input: *const fa_tensor_arg,
        output: *const fa_tensor_arg,
        params: *const fa_kv_rearrange_params,
    ) -> fa_status;
    pub fn fa_repeat_kv_heads(
        ctx: *mut fa_ctx,
        input: *const fa_tensor_arg,
        output: *const fa_tensor_arg,
        params: *const fa_repeat_kv_heads_params,
    ) -> fa_status;
    pub fn fa_sdpa_reference(
        ctx: *mut fa_ctx,
        q: *const fa_tensor_arg,
        k: *const fa_tensor_arg,
        v: *const fa_tensor_arg,
        output: *const fa_tensor_arg,
        causal: c_int,
        query_offset: u32,
        n_heads: u32,
        head_dim: u32,
        kv_seq_len: u32,
        m: u32,
        kv_head_major: c_int,
    ) -> fa_status;
    pub fn fa_measure_clock(
        ctx: *mut fa_ctx,
        matrix_load: c_int,
        iterations: u32,
        shader_mhz: *mut f32,
        busy_ms: *mut f32,
    ) -> fa_status;
    pub fn fa_version() -> *const c_char;
    pub fn fa_device_info(
        ctx: *mut fa_ctx,
        name_out: *mut c_char,
        name_cap: usize,
        compute_units: *mut u32,
        global_mem_bytes: *mut u64,
    ) -> fa_status;
    pub fn fa_device_mem_info(ctx: *mut fa_ctx, free_bytes: *mut u64, total_bytes: *mut u64) -> fa_status;
}
