//! Raw declarations of `libophip.so` (`include/ophip.h`), the C ABI of the MI355X backend.
//! Field order and types mirror the header one to one; nothing here owns anything.
#![allow(non_camel_case_types)]

use std::ffi::{c_char, c_int, c_uint, c_void};

pub type ophip_stream = *mut c_void;

#[repr(C)]
pub struct ophip_device {
    _opaque: [u8; 0],
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct ophip_config {
    pub low_diversity_cache: usize,
    pub medium_diversity_cache: usize,
    pub high_diversity_cache: usize,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct ophip_device_info {
    pub name: [c_char; 64],
    pub arch: [c_char; 32],
    pub compute_units: c_int,
    pub wavefront_size: c_int,
    pub max_threads_per_block: c_int,
    pub lds_per_block: usize,
    pub total_memory: usize,
    pub clock_khz: c_int,
}

/// `[dt][ndim][shape..][strides..]` of a `TensorLayout`, borrowed.
#[repr(C)]
#[derive(Clone, Copy)]
pub struct ophip_tensor_layout {
    pub dt: u64,
    pub ndim: u64,
    pub shape: *const usize,
    pub strides: *const isize,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct ophip_queue_alloc {
    pub ctx: *mut c_void,
    pub stream: ophip_stream,
    pub alloc: extern "C" fn(*mut c_void, usize) -> *mut c_void,
    pub free: extern "C" fn(*mut c_void, *mut c_void),
}

#[repr(C)]
pub struct ophip_rms_norm_args {
    pub y_layout: ophip_tensor_layout,
    pub y_base: *mut c_void,
    pub x_layout: ophip_tensor_layout,
    pub x_base: *const c_void,
    pub w_layout: ophip_tensor_layout,
    pub w_base: *const c_void,
    pub epsilon: f32,
}

#[repr(C)]
pub struct ophip_rope_args {
    pub t_layout: ophip_tensor_layout,
    pub t_base: *mut c_void,
    pub p_layout: ophip_tensor_layout,
    pub p_base: *const c_void,
    pub sin_layout: ophip_tensor_layout,
    pub sin_base: *const c_void,
    pub cos_layout: ophip_tensor_layout,
    pub cos_base: *const c_void,
    pub theta: f32,
}

#[repr(C)]
pub struct ophip_fused_softmax_args {
    pub att_mask: u8,
    pub att_layout: ophip_tensor_layout,
    pub att_base: *mut c_void,
}

#[repr(C)]
pub struct ophip_rearrange_args {
    pub dst_layout: ophip_tensor_layout,
    pub dst_base: *mut c_void,
    pub src_layout: ophip_tensor_layout,
    pub src_base: *const c_void,
}

#[repr(C)]
pub struct ophip_swiglu_args {
    pub gate_layout: ophip_tensor_layout,
    pub gate_base: *mut c_void,
    pub up_layout: ophip_tensor_layout,
    pub up_base: *const c_void,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct ophip_sample_args {
    pub temperature: f32,
    pub top_p: f32,
    pub top_k: usize,
}

#[repr(C)]
pub struct ophip_random_sample_args {
    pub kv_pair: ophip_tensor_layout,
    pub kv_pair_base: *mut c_void,
    pub logits: ophip_tensor_layout,
    pub logits_base: *const c_void,
    pub indices: ophip_tensor_layout,
    pub indices_base: *const c_void,
    pub config: ophip_sample_args,
    pub seed: f32,
}

#[repr(C)]
pub struct ophip_mat_mul_args {
    pub c_layout: ophip_tensor_layout,
    pub c_base: *mut c_void,
    pub beta: f32,
    pub a_layout: ophip_tensor_layout,
    pub a_base: *const c_void,
    pub b_layout: ophip_tensor_layout,
    pub b_base: *const c_void,
    pub alpha: f32,
}

#[repr(C)]
pub struct ophip_layer_norm_args {
    pub y_layout: ophip_tensor_layout,
    pub y_base: *mut c_void,
    pub x_layout: ophip_tensor_layout,
    pub x_base: *const c_void,
    pub scale_layout: ophip_tensor_layout,
    pub scale_base: *const c_void,
    pub bias_layout: ophip_tensor_layout,
    pub bias_base: *const c_void,
    pub epsilon: f32,
}

#[repr(C)]
pub struct ophip_gelu_args {
    pub layout: ophip_tensor_layout,
    pub base: *mut c_void,
}

#[repr(C)]
pub struct ophip_add_args {
    pub c_layout: ophip_tensor_layout,
    pub c_base: *mut c_void,
    pub a_layout: ophip_tensor_layout,
    pub a_base: *const c_void,
    pub b_layout: ophip_tensor_layout,
    pub b_base: *const c_void,
}

#[repr(C)]
pub struct ophip_add_rows_args {
    pub dst_layout: ophip_tensor_layout,
    pub dst_base: *mut c_void,
    pub src_layout: ophip_tensor_layout,
    pub src_base: *const c_void,
    pub idx_layout: ophip_tensor_layout,
    pub idx_base: *const c_void,
}

/// Declares the opaque operator type and its four verbs (create / scheme / launch / destroy).
macro_rules! verbs {
    ($($op:ident, $args:ident, $create:ident, $scheme:ident, $launch:ident, $destroy:ident;)*) => {
        $(
            #[repr(C)]
            pub struct $op { _opaque: [u8; 0] }
        )*
        #[link(name = "ophip")]
        extern "C" {
            $(
                pub fn $create(dev: *mut ophip_device, out: *mut *mut $op) -> c_int;
                pub fn $scheme(op: *mut $op, args: *const $args, max_workspace_size: usize, workspace_size: *mut usize) -> c_int;
                pub fn $launch(op: *const $op, args: *const $args, workspace: *mut c_void, workspace_len: usize,
                               queue_alloc: *const ophip_queue_alloc) -> c_int;
                pub fn $destroy(op: *mut $op);
            )*
        }
    };
}

verbs! {
    ophip_rms_norm, ophip_rms_norm_args, ophip_rms_norm_create, ophip_rms_norm_scheme, ophip_rms_norm_launch, ophip_rms_norm_destroy;
    ophip_rope, ophip_rope_args, ophip_rope_create, ophip_rope_scheme, ophip_rope_launch, ophip_rope_destroy;
    ophip_fused_softmax, ophip_fused_softmax_args, ophip_fused_softmax_create, ophip_fused_softmax_scheme, ophip_fused_softmax_launch, ophip_fused_softmax_destroy;
    ophip_rearrange, ophip_rearrange_args, ophip_rearrange_create, ophip_rearrange_scheme, ophip_rearrange_launch, ophip_rearrange_destroy;
    ophip_swiglu, ophip_swiglu_args, ophip_swiglu_create, ophip_swiglu_scheme, ophip_swiglu_launch, ophip_swiglu_destroy;
    ophip_random_sample, ophip_random_sample_args, ophip_random_sample_create, ophip_random_sample_scheme, ophip_random_sample_launch, ophip_random_sample_destroy;
    ophip_mat_mul, ophip_mat_mul_args, ophip_mat_mul_create, ophip_mat_mul_scheme, ophip_mat_mul_launch, ophip_mat_mul_destroy;
    ophip_layer_norm, ophip_layer_norm_args, ophip_layer_norm_create, ophip_layer_norm_scheme, ophip_layer_norm_launch, ophip_layer_norm_destroy;
    ophip_gelu, ophip_gelu_args, ophip_gelu_create, ophip_gelu_scheme, ophip_gelu_launch, ophip_gelu_destroy;
    ophip_add, ophip_add_args, ophip_add_create, ophip_add_scheme, ophip_add_launch, ophip_add_destroy;
    ophip_add_rows, ophip_add_rows_args, ophip_add_rows_create, ophip_add_rows_scheme, ophip_add_rows_launch, ophip_add_rows_destroy;
}

#[link(name = "ophip")]
extern "C" {
    pub fn ophip_last_error() -> *const c_char;
    pub fn ophip_device_count() -> c_int;
    pub fn ophip_device_create(ordinal: c_int, cfg: *const ophip_config, out: *mut *mut ophip_device) -> c_int;
    pub fn ophip_device_release(dev: *mut ophip_device);
    pub fn ophip_device_get_info(dev: *const ophip_device, out: *mut ophip_device_info) -> c_int;
    pub fn ophip_malloc(dev: *mut ophip_device, size: usize, out: *mut *mut c_void) -> c_int;
    pub fn ophip_free(dev: *mut ophip_device, ptr: *mut c_void) -> c_int;
    pub fn ophip_memcpy_h2d(dev: *mut ophip_device, dst: *mut c_void, src: *const c_void, size: usize, stream: ophip_stream) -> c_int;
    pub fn ophip_memcpy_d2h(dev: *mut ophip_device, dst: *mut c_void, src: *const c_void, size: usize, stream: ophip_stream) -> c_int;
    pub fn ophip_memcpy_d2d(dev: *mut ophip_device, dst: *mut c_void, src: *const c_void, size: usize, stream: ophip_stream) -> c_int;
    pub fn ophip_stream_create(dev: *mut ophip_device, out: *mut ophip_stream) -> c_int;
    pub fn ophip_stream_destroy(dev: *mut ophip_device, stream: ophip_stream) -> c_int;
    pub fn ophip_stream_synchronize(dev: *mut ophip_device, stream: ophip_stream) -> c_int;
    pub fn ophip_queue_alloc_from_stream(dev: *mut ophip_device, stream: ophip_stream, out: *mut ophip_queue_alloc) -> c_int;
}

// ---- the rest of include/ophip.h: everything the header declares is declared here too -------------
#[repr(C)]
pub struct ophip_mem_pool {
    _opaque: [u8; 0],
}
#[repr(C)]
pub struct ophip_offset_calculator {
    _opaque: [u8; 0],
}
#[repr(C)]
pub struct ophip_attention {
    _opaque: [u8; 0],
}
#[repr(C)]
pub struct ophip_attention_kv_cached {
    _opaque: [u8; 0],
}
#[repr(C)]
pub struct ophip_conv {
    _opaque: [u8; 0],
}
#[repr(C)]
#[derive(Clone, Copy)]
pub struct ophip_rope_seq {
    pub pos: usize,
    pub len: usize,
}
#[repr(C)]
#[derive(Clone, Copy)]
pub struct ophip_kv_pair {
    pub idx: u32,
    pub val: u32,
}
#[repr(C)]
#[derive(Clone, Copy)]
pub struct ophip_mat_mul_layout {
    pub dt: u64,
    pub ab_swap: i32,
    pub a_trans: i32,
    pub b_trans: i32,
    pub _pad: i32,
    pub batch: usize,
    pub m: usize,
    pub n: usize,
    pub k: usize,
    pub c_stride: isize,
    pub c_ld: isize,
    pub a_stride: isize,
    pub a_ld: isize,
    pub b_stride: isize,
    pub b_ld: isize,
}
#[repr(C)]
#[derive(Clone, Copy)]
pub struct ophip_attention_args {
    pub q_layout: ophip_tensor_layout,
    pub q_base: *mut c_void,
    pub k_layout: ophip_tensor_layout,
    pub k_base: *const c_void,
    pub v_layout: ophip_tensor_layout,
    pub v_base: *const c_void,
    pub o_layout: ophip_tensor_layout,
    pub o_base: *mut c_void,
    pub mask: u8,
}
#[repr(C)]
#[derive(Clone, Copy)]
pub struct ophip_attention_kv_cached_args {
    pub q_layout: ophip_tensor_layout,
    pub q_base: *mut c_void,
    pub k_layout: ophip_tensor_layout,
    pub k_base: *const c_void,
    pub v_layout: ophip_tensor_layout,
    pub v_base: *const c_void,
    pub o_layout: ophip_tensor_layout,
    pub o_base: *mut c_void,
    pub k_cache_layout: ophip_tensor_layout,
    pub k_cache_base: *mut c_void,
    pub v_cache_layout: ophip_tensor_layout,
    pub v_cache_base: *mut c_void,
    pub mask: u8,
    pub pos: usize,
}
#[repr(C)]
#[derive(Clone, Copy)]
pub struct ophip_conv_args {
    pub y_layout: ophip_tensor_layout,
    pub y_base: *mut c_void,
    pub x_layout: ophip_tensor_layout,
    pub x_base: *const c_void,
    pub w_layout: ophip_tensor_layout,
    pub w_base: *const c_void,
    pub b_layout: ophip_tensor_layout,
    pub b_base: *const c_void,
    pub strides: [usize; 2],
    pub dilations: [usize; 2],
    pub pads: [usize; 4],
}
#[link(name = "ophip")]
extern "C" {
    pub fn ophip_status_name(status: c_int) -> *const c_char;
    pub fn ophip_dtype_nbytes(dt: u64) -> usize;
    pub fn ophip_device_retain(dev: *mut ophip_device);
    pub fn ophip_memset(dev: *mut ophip_device, dst: *mut c_void, value: c_int, size: usize, stream: *mut c_void) -> c_int;
    pub fn ophip_event_create(dev: *mut ophip_device, out: *mut *mut c_void) -> c_int;
    pub fn ophip_event_destroy(dev: *mut ophip_device, ev: *mut c_void) -> c_int;
    pub fn ophip_event_record(dev: *mut ophip_device, ev: *mut c_void, stream: *mut c_void) -> c_int;
    pub fn ophip_event_synchronize(dev: *mut ophip_device, ev: *mut c_void) -> c_int;
    pub fn ophip_event_elapsed_ms(dev: *mut ophip_device, start: *mut c_void, stop: *mut c_void, ms: *mut f32) -> c_int;
    pub fn ophip_time_next_launch(dev: *mut ophip_device, stream: *mut c_void, start: *mut c_void, stop: *mut c_void) -> c_int;

    pub fn ophip_stream_begin_capture(dev: *mut ophip_device, stream: *mut c_void) -> c_int;
    pub fn ophip_stream_end_capture(dev: *mut ophip_device, stream: *mut c_void, out: *mut *mut c_void) -> c_int;
    pub fn ophip_graph_launch(dev: *mut ophip_device, graph: *mut c_void, stream: *mut c_void) -> c_int;
    pub fn ophip_graph_destroy(dev: *mut ophip_device, graph: *mut c_void) -> c_int;
    pub fn ophip_mem_pool_create(dev: *mut ophip_device, stream: *mut c_void, out: *mut *mut ophip_mem_pool) -> c_int;
    pub fn ophip_mem_pool_put(pool: *mut ophip_mem_pool, size: usize) -> c_int;
    pub fn ophip_mem_pool_queue_alloc(pool: *mut ophip_mem_pool, out: *mut ophip_queue_alloc) -> c_int;
    pub fn ophip_mem_pool_destroy(pool: *mut ophip_mem_pool);
    pub fn ophip_offset_calculator_create(alignment: usize) -> *mut ophip_offset_calculator;
    pub fn ophip_offset_calculator_destroy(c: *mut ophip_offset_calculator);
    pub fn ophip_offset_calculator_put(c: *mut ophip_offset_calculator, start: usize, end: usize);
    pub fn ophip_offset_calculator_take(c: *mut ophip_offset_calculator, size: usize, start: *mut usize,
        end: *mut usize) -> c_int;
    pub fn ophip_rope_build_pos(dt: u64, nt: usize, seqs: *const ophip_rope_seq, nseq: usize,
        queue_alloc: *const ophip_queue_alloc, out: *mut *mut c_void) -> c_int;
    pub fn ophip_rope_build_sincos(dt: u64, nctx: usize, dh: usize, queue_alloc: *const ophip_queue_alloc,
        nctx_out: *mut usize, out: *mut *mut c_void) -> c_int;
    pub fn ophip_rearrange_plan(args: *const ophip_rearrange_args, out: *mut isize, ndim_out: *mut usize) -> c_int;
    pub fn ophip_sample_args_new(temperature: f32, top_p: f32, top_k: usize, out: *mut ophip_sample_args) -> c_int;
    pub fn ophip_sample_args_argmax() -> ophip_sample_args;
    pub fn ophip_random_sample_launch_batch(op: *const ophip_random_sample, args: *const ophip_random_sample_args,
        rows: usize, row_stride: isize, seeds: *const f32, workspace: *mut c_void, workspace_len: usize,
        queue_alloc: *const ophip_queue_alloc) -> c_int;
    pub fn ophip_random_sample_build_indices(n: usize, queue_alloc: *const ophip_queue_alloc, out: *mut *mut c_void) -> c_int;
    pub fn ophip_mat_mul_plan(args: *const ophip_mat_mul_args, out: *mut ophip_mat_mul_layout) -> c_int;
    pub fn ophip_mat_mul_launch_static(op: *const ophip_mat_mul, args: *const ophip_mat_mul_args,
        stream: *mut c_void) -> c_int;
    pub fn ophip_mat_mul_describe(op: *const ophip_mat_mul, args: *const ophip_mat_mul_args, out: *mut c_char,
        len: usize) -> c_int;
    pub fn ophip_attention_create(dev: *mut ophip_device, out: *mut *mut ophip_attention) -> c_int;
    pub fn ophip_attention_scheme(op: *mut ophip_attention, args: *const ophip_attention_args,
        max_workspace_size: usize, workspace_size: *mut usize) -> c_int;
    pub fn ophip_attention_launch(op: *const ophip_attention, args: *const ophip_attention_args,
        workspace: *mut c_void, workspace_len: usize, queue_alloc: *const ophip_queue_alloc) -> c_int;
    pub fn ophip_attention_destroy(op: *mut ophip_attention);
    pub fn ophip_attention_kv_cached_create(dev: *mut ophip_device, out: *mut *mut ophip_attention_kv_cached) -> c_int;
    pub fn ophip_attention_kv_cached_scheme(op: *mut ophip_attention_kv_cached,
        args: *const ophip_attention_kv_cached_args, max_workspace_size: usize, workspace_size: *mut usize) -> c_int;
    pub fn ophip_attention_kv_cached_launch(op: *const ophip_attention_kv_cached,
        args: *const ophip_attention_kv_cached_args, workspace: *mut c_void, workspace_len: usize,
        queue_alloc: *const ophip_queue_alloc) -> c_int;
    pub fn ophip_attention_kv_cached_destroy(op: *mut ophip_attention_kv_cached);
    pub fn ophip_add_plan(args: *const ophip_add_args, out: *mut isize, ndim_out: *mut usize) -> c_int;
    pub fn ophip_conv_create(dev: *mut ophip_device, out: *mut *mut ophip_conv) -> c_int;
    pub fn ophip_conv_scheme(op: *mut ophip_conv, args: *const ophip_conv_args, max_workspace_size: usize,
        workspace_size: *mut usize) -> c_int;
    pub fn ophip_conv_launch(op: *const ophip_conv, args: *const ophip_conv_args, workspace: *mut c_void,
        workspace_len: usize, queue_alloc: *const ophip_queue_alloc) -> c_int;
    pub fn ophip_conv_destroy(op: *mut ophip_conv);
}
