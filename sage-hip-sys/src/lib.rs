//! Raw bindings to `libsage_hip.so`: `include/sage_hip.h` declaration for declaration, in the header's order.
//!
//! This is the crate the reference would depend on to reach the gfx950 backend from its operators'
//! `compute` methods (`src/ops.rs:79-101`) and from a `Data::Hip` storage variant next to
//! `Data::{Host,OpenCl,Cuda}` (`src/tensor.rs:569-574`).  Nothing here is safe Rust: every function takes
//! raw pointers and returns an `sg_status` code; the safe layer (descriptor construction from `Tensor`,
//! status -> `Error` mapping) belongs to the reference side.
//!
//! A test of the repository that holds this file parses both this file and the header and fails when the
//! entry points, their argument lists, the struct fields or the constants differ.
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_int, c_void};

pub const SG_MAX_RANK: usize = 8;
pub const SG_MAX_MAP_INPUTS: usize = 16;
pub const SG_MAX_EXPR: usize = 128;
/// Allocator capacity a default reference `Context` runs with: 1000 MiB (`session/context.rs:49`).
pub const SG_REFERENCE_CAPACITY_BYTES: u64 = 1000 * 1024 * 1024;
/// Size of the static per-GPU split-K workspace `sg_gemm_noalloc` uses.
pub const SG_GEMM_NOALLOC_SCRATCH_BYTES: u32 = 32 << 20;

// sg_status
pub const SG_OK: c_int = 0;
pub const SG_ERR_OOM: c_int = 1;
pub const SG_ERR_DEVICE: c_int = 2;
pub const SG_ERR_SHAPE: c_int = 3;
pub const SG_ERR_DTYPE: c_int = 4;
pub const SG_ERR_ARG: c_int = 5;

// sg_dtype: the order of the reference's `DataType` (`tensor/data.rs:14-30`), so `data_type as i32` is the code
pub const SG_CHAR: i32 = 0;
pub const SG_SHORT: i32 = 1;
pub const SG_INT: i32 = 2;
pub const SG_LONG: i32 = 3;
pub const SG_UCHAR: i32 = 4;
pub const SG_USHORT: i32 = 5;
pub const SG_UINT: i32 = 6;
pub const SG_ULONG: i32 = 7;
pub const SG_FLOAT: i32 = 8;
pub const SG_HALF: i32 = 9;

// sg_unary: the order of `UnaryMap` (`ops/map.rs:93-130`)
pub const SG_U_COPY: i32 = 0;
pub const SG_U_ABS: i32 = 1;
pub const SG_U_NEG: i32 = 2;
pub const SG_U_RECIP: i32 = 3;
pub const SG_U_LOG: i32 = 4;
pub const SG_U_EXP: i32 = 5;
pub const SG_U_SQRT: i32 = 6;
pub const SG_U_SQUARE: i32 = 7;
pub const SG_U_ERF: i32 = 8;
pub const SG_U_SIGN: i32 = 9;
pub const SG_U_CEIL: i32 = 10;
pub const SG_U_FLOOR: i32 = 11;
pub const SG_U_ROUND: i32 = 12;
pub const SG_U_SIN: i32 = 13;
pub const SG_U_SINH: i32 = 14;
pub const SG_U_COS: i32 = 15;
pub const SG_U_COSH: i32 = 16;
pub const SG_U_TAN: i32 = 17;
pub const SG_U_TANH: i32 = 18;
pub const SG_U_ASIN: i32 = 19;
pub const SG_U_ASINH: i32 = 20;
pub const SG_U_ACOS: i32 = 21;
pub const SG_U_ACOSH: i32 = 22;
pub const SG_U_ATAN: i32 = 23;
pub const SG_U_ATANH: i32 = 24;
pub const SG_U_NOT: i32 = 25;
pub const SG_U_CAST_INT: i32 = 26;
pub const SG_U_CAST_FLOAT: i32 = 27;
pub const SG_U__COUNT: i32 = 28;

// sg_binary: the order of `BinaryMap` (`ops/map.rs:152-172`)
pub const SG_B_ADD: i32 = 0;
pub const SG_B_SUB: i32 = 1;
pub const SG_B_DIV: i32 = 2;
pub const SG_B_MUL: i32 = 3;
pub const SG_B_MOD: i32 = 4;
pub const SG_B_POW: i32 = 5;
pub const SG_B_MIN: i32 = 6;
pub const SG_B_MAX: i32 = 7;
pub const SG_B_AND: i32 = 8;
pub const SG_B_OR: i32 = 9;
pub const SG_B_EQ: i32 = 10;
pub const SG_B_NE: i32 = 11;
pub const SG_B_GT: i32 = 12;
pub const SG_B_GE: i32 = 13;
pub const SG_B_LT: i32 = 14;
pub const SG_B_LE: i32 = 15;
pub const SG_B__COUNT: i32 = 16;

// sg_ternary
pub const SG_T_COND: i32 = 0;
pub const SG_T__COUNT: i32 = 1;

// sg_expr_kind
pub const SG_EXPR_INPUT: i32 = 0;
pub const SG_EXPR_LITERAL: i32 = 1;
pub const SG_EXPR_UNARY: i32 = 2;
pub const SG_EXPR_BINARY: i32 = 3;
pub const SG_EXPR_TERNARY: i32 = 4;

// sg_reduce_op, sg_reduce_arg_op, sg_reduce_init
pub const SG_R_SUM: c_int = 0;
pub const SG_R_PROD: c_int = 1;
pub const SG_R_MAX: c_int = 2;
pub const SG_R_MIN: c_int = 3;
pub const SG_RA_MAX: c_int = 0;
pub const SG_RA_MIN: c_int = 1;
pub const SG_INIT_REF_ZERO: c_int = 0;
pub const SG_INIT_IDENTITY: c_int = 1;

// sg_act
pub const SG_ACT_NONE: i32 = 0;
pub const SG_ACT_RELU: i32 = 1;
pub const SG_ACT_GELU_ERF: i32 = 2;

/// `TensorDesc` + `Shape` (`tensor.rs:38-41`, `shape.rs:38-42`) plus the device pointer of the buffer.
#[repr(C)]
#[derive(Clone, Copy)]
pub struct sg_tensor {
    pub base: *mut c_void,
    pub dtype: i32,
    pub rank: i32,
    pub extents: [i64; SG_MAX_RANK],
    pub strides: [i64; SG_MAX_RANK],
    pub offset: i64,
}

/// One element of `VariadicMapOperator.expr` (`map.rs:199-222`), prefix order.
#[repr(C)]
#[derive(Clone, Copy)]
pub struct sg_expr {
    pub kind: i32,
    pub op: i32,
    pub dtype: i32,
    pub bits: u32,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct sg_gemm_epilogue {
    pub alpha: f32,
    pub act: i32,
    pub act_post: i32,
    pub bias: *const sg_tensor,
    pub residual: *const sg_tensor,
}

/// Scalars of `Adam` (`optim.rs:98-127`); `one_minus_beta*` are the f32 differences `1.0 - self.beta*`.
#[repr(C)]
#[derive(Clone, Copy)]
pub struct sg_adam_hyper {
    pub lr: f32,
    pub beta1: f32,
    pub beta2: f32,
    pub one_minus_beta1: f32,
    pub one_minus_beta2: f32,
    pub eps: f32,
    pub weight_decay: f32,
}

/// Opaque: one device, one in-order stream, the kernel cache and the allocator.
#[repr(C)]
pub struct sg_ctx {
    _private: [u8; 0],
}

/// Opaque: a recorded launch sequence.
#[repr(C)]
pub struct sg_graph {
    _private: [u8; 0],
}

extern "C" {
    // ---- context, memory, transfers
    pub fn sg_ctx_create(device_idx: c_int, capacity_bytes: u64, out: *mut *mut sg_ctx) -> c_int;
    pub fn sg_ctx_create_pooled(device_idx: c_int, capacity_bytes: u64, use_cache: c_int, use_sub_buffer: c_int, out: *mut *mut sg_ctx) -> c_int;
    pub fn sg_ctx_destroy(ctx: *mut sg_ctx) -> c_int;
    pub fn sg_alloc(ctx: *mut sg_ctx, nbytes: u64, dptr: *mut *mut c_void) -> c_int;
    pub fn sg_free(ctx: *mut sg_ctx, dptr: *mut c_void) -> c_int;
    pub fn sg_trim(ctx: *mut sg_ctx) -> c_int;
    pub fn sg_mem_stats(ctx: *mut sg_ctx, used: *mut u64, reserved: *mut u64, peak: *mut u64, capacity: *mut u64) -> c_int;
    pub fn sg_memcpy_h2d(ctx: *mut sg_ctx, dst_dev: *mut c_void, src_host: *const c_void, nbytes: u64) -> c_int;
    pub fn sg_memcpy_d2h(ctx: *mut sg_ctx, dst_host: *mut c_void, src_dev: *const c_void, nbytes: u64) -> c_int;
    pub fn sg_memcpy_d2d(ctx: *mut sg_ctx, dst_dev: *mut c_void, src_dev: *const c_void, nbytes: u64) -> c_int;
    pub fn sg_fill_u32(ctx: *mut sg_ctx, dst_dev: *mut c_void, pattern: u32, count: u64) -> c_int;
    pub fn sg_sync(ctx: *mut sg_ctx) -> c_int;
    pub fn sg_stream(ctx: *mut sg_ctx) -> *mut c_void;
    pub fn sg_event_create(ctx: *mut sg_ctx, event: *mut *mut c_void) -> c_int;
    pub fn sg_event_record(ctx: *mut sg_ctx, event: *mut c_void) -> c_int;
    pub fn sg_event_elapsed_ms(ctx: *mut sg_ctx, start: *mut c_void, stop: *mut c_void, ms: *mut f32) -> c_int;
    pub fn sg_event_destroy(ctx: *mut sg_ctx, event: *mut c_void) -> c_int;
    pub fn sg_last_error(ctx: *mut sg_ctx) -> *const c_char;
    pub fn sg_last_oom(ctx: *mut sg_ctx, needed: *mut u64, total: *mut u64) -> c_int;
    pub fn sg_kernel_cache_size(ctx: *mut sg_ctx) -> c_int;

    // ---- fused elementwise maps
    pub fn sg_map(ctx: *mut sg_ctx, prog: *const sg_expr, n_prog: c_int, inputs: *const sg_tensor, n_in: c_int,
                  out: *const sg_tensor) -> c_int;
    pub fn sg_map_source(ctx: *mut sg_ctx, prog: *const sg_expr, n_prog: c_int, inputs: *const sg_tensor, n_in: c_int,
                         out: *const sg_tensor, buf: *mut c_char, cap: u64, result_dtype: *mut i32) -> c_int;
    pub fn sg_map_compile_only(source: *const c_char, log_buf: *mut c_char, log_cap: u64) -> c_int;

    // ---- reductions
    pub fn sg_reduce(ctx: *mut sg_ctx, op: c_int, axes: *const i32, n_axes: c_int, init_mode: c_int,
                     input: *const sg_tensor, out: *const sg_tensor) -> c_int;
    pub fn sg_reduce_arg(ctx: *mut sg_ctx, op: c_int, axis: c_int, input: *const sg_tensor, out: *const sg_tensor) -> c_int;

    // ---- indexing kernels
    pub fn sg_gather(ctx: *mut sg_ctx, axis: c_int, x: *const sg_tensor, ind: *const sg_tensor, out: *const sg_tensor) -> c_int;
    pub fn sg_scatter(ctx: *mut sg_ctx, axis: c_int, x: *const sg_tensor, ind: *const sg_tensor, out: *const sg_tensor) -> c_int;
    pub fn sg_unslice(ctx: *mut sg_ctx, axis: c_int, start: i64, x: *const sg_tensor, out: *const sg_tensor) -> c_int;
    pub fn sg_concat(ctx: *mut sg_ctx, axis: c_int, inputs: *const sg_tensor, n_in: c_int, out: *const sg_tensor) -> c_int;

    // ---- GEMM
    pub fn sg_gemm(ctx: *mut sg_ctx, transpose_a: c_int, transpose_b: c_int, a: *const sg_tensor, b: *const sg_tensor,
                   c: *const sg_tensor, epi: *const sg_gemm_epilogue) -> c_int;
    pub fn sg_gemm_noalloc(ctx: *mut sg_ctx, transpose_a: c_int, transpose_b: c_int, a: *const sg_tensor,
                           b: *const sg_tensor, c: *const sg_tensor, epi: *const sg_gemm_epilogue) -> c_int;
    pub fn sg_gemm_batched(ctx: *mut sg_ctx, transpose_a: c_int, transpose_b: c_int, a: *const sg_tensor,
                           b: *const sg_tensor, c: *const sg_tensor, epi: *const sg_gemm_epilogue) -> c_int;
    pub fn sg_matmul_strided(ctx: *mut sg_ctx, a: *const sg_tensor, b: *const sg_tensor, c: *const sg_tensor,
                             epi: *const sg_gemm_epilogue) -> c_int;
    pub fn sg_gemm_last_kernel_name(ctx: *mut sg_ctx, buf: *mut c_char, cap: u64) -> c_int;

    // ---- convolution feeder, pooling
    pub fn sg_im2col(ctx: *mut sg_ctx, x: *const sg_tensor, out: *const sg_tensor, ker: *const i32, stride: *const i32,
                     pad: *const i32, dil: *const i32) -> c_int;
    pub fn sg_conv2d(ctx: *mut sg_ctx, x: *const sg_tensor, filter: *const sg_tensor, out: *const sg_tensor,
                     stride: *const i32, pad: *const i32, dil: *const i32, epi: *const sg_gemm_epilogue) -> c_int;
    pub fn sg_pool2d(ctx: *mut sg_ctx, op: c_int, init_mode: c_int, x: *const sg_tensor, out: *const sg_tensor,
                     ker: *const i32, stride: *const i32, pad: *const i32, dil: *const i32) -> c_int;
    pub fn sg_col2im(ctx: *mut sg_ctx, x: *const sg_tensor, out: *const sg_tensor, ker: *const i32, stride: *const i32,
                     pad: *const i32, dil: *const i32) -> c_int;

    // ---- random fills
    pub fn sg_rand_uniform(ctx: *mut sg_ctx, seed_x: u32, seed_y: u32, out: *const sg_tensor) -> c_int;
    pub fn sg_rand_normal(ctx: *mut sg_ctx, seed_x: u32, seed_y: u32, out: *const sg_tensor) -> c_int;

    // ---- optimizer step
    pub fn sg_adam_update(ctx: *mut sg_ctx, n_tensors: c_int, values: *const sg_tensor, grads: *const sg_tensor,
                          m: *const sg_tensor, v: *const sg_tensor, step: *const sg_tensor, h: *const sg_adam_hyper) -> c_int;

    // ---- fused row operators, attention
    pub fn sg_softmax_lastaxis(ctx: *mut sg_ctx, x: *const sg_tensor, addend: *const sg_tensor, out: *const sg_tensor) -> c_int;
    pub fn sg_softmax_cross_entropy(ctx: *mut sg_ctx, logits: *const sg_tensor, labels: *const sg_tensor,
                                    loss: *const sg_tensor) -> c_int;
    pub fn sg_layer_norm_lastaxis(ctx: *mut sg_ctx, x: *const sg_tensor, gamma: *const sg_tensor, beta: *const sg_tensor,
                                  eps: f32, out: *const sg_tensor) -> c_int;
    pub fn sg_attention(ctx: *mut sg_ctx, q: *const sg_tensor, k: *const sg_tensor, v: *const sg_tensor,
                        addend: *const sg_tensor, scale: f32, out: *const sg_tensor) -> c_int;

    // ---- replay of a recorded launch sequence
    pub fn sg_graph_begin(ctx: *mut sg_ctx) -> c_int;
    pub fn sg_graph_end(ctx: *mut sg_ctx, out: *mut *mut sg_graph) -> c_int;
    pub fn sg_graph_launch(ctx: *mut sg_ctx, graph: *mut sg_graph) -> c_int;
    pub fn sg_graph_destroy(ctx: *mut sg_ctx, graph: *mut sg_graph) -> c_int;
}
