//! Raw bindings to `libcybq.so`: one `extern "C"` declaration per entry point of
//! `include/cybq.h`, same order, same argument names.  Pointers named `x`, `y`, `out`,
//! `residual`, `gamma`, `src`, `q_out`, `scales_out`, `q_dev`, `scales_dev` are DEVICE
//! pointers; `q` / `scales` of `cybq_weight_upload` are host pointers (the mmap'd `.model`
//! file).  `stream` is a `hipStream_t` (null = the default stream).  Every function returns
//! `CYBQ_OK` (0) or a negative status; nothing unwinds across the boundary.
#![allow(non_camel_case_types)]

use core::ffi::{c_char, c_float, c_int, c_void};

#[repr(C)]
pub struct cybq_ctx {
    _opaque: [u8; 0],
}
#[repr(C)]
pub struct cybq_weight {
    _opaque: [u8; 0],
}

pub const CYBQ_GROUP: c_int = 32;

// enum cybq_status
pub const CYBQ_OK: c_int = 0;
pub const CYBQ_ERR_INVALID: c_int = -1;
pub const CYBQ_ERR_SHAPE: c_int = -2;
pub const CYBQ_ERR_ALIGN: c_int = -3;
pub const CYBQ_ERR_NO_DEVICE: c_int = -4;
pub const CYBQ_ERR_HIP: c_int = -5;
pub const CYBQ_ERR_NOMEM: c_int = -6;
pub const CYBQ_ERR_UNSUPPORTED: c_int = -7;

// enum cybq_quant
pub const CYBQ_Q4: c_int = 4;
pub const CYBQ_Q8: c_int = 8;
// enum cybq_layout
pub const CYBQ_LAYOUT_PLANAR: c_int = 0;
pub const CYBQ_LAYOUT_BLOCK_AOS: c_int = 1;
// enum cybq_dtype
pub const CYBQ_F32: c_int = 0;
pub const CYBQ_F16: c_int = 1;
pub const CYBQ_BF16: c_int = 2;
// enum cybq_prefill_mode
pub const CYBQ_PREFILL_FAST: c_int = 0;
pub const CYBQ_PREFILL_EXACT: c_int = 1;
// enum cybq_decode_mode
pub const CYBQ_DECODE_STREAM: c_int = 0;
pub const CYBQ_DECODE_EXACT: c_int = 1;
// enum cybq_epilogue
pub const CYBQ_EPI_NONE: c_int = 0;
pub const CYBQ_EPI_ADD: c_int = 1;
pub const CYBQ_EPI_SWIGLU: c_int = 2;

extern "C" {
    pub fn cybq_init(device: c_int, out: *mut *mut cybq_ctx) -> c_int;
    pub fn cybq_destroy(ctx: *mut cybq_ctx);
    pub fn cybq_strerror(status: c_int) -> *const c_char;
    pub fn cybq_last_error(ctx: *const cybq_ctx) -> *const c_char;
    pub fn cybq_version() -> *const c_char;

    pub fn cybq_weight_upload(ctx: *mut cybq_ctx, quant: c_int, layout: c_int, N: i64, K: i64, q: *const c_void,
                              scales: *const c_void, out: *mut *mut cybq_weight) -> c_int;
    pub fn cybq_weight_clone(ctx: *mut cybq_ctx, src: *const cybq_weight, out: *mut *mut cybq_weight) -> c_int;
    pub fn cybq_weight_free(ctx: *mut cybq_ctx, w: *mut cybq_weight) -> c_int;
    pub fn cybq_weight_info(w: *const cybq_weight, quant: *mut c_int, N: *mut i64, K: *mut i64,
                            device_bytes: *mut i64) -> c_int;

    pub fn cybq_matmul(ctx: *mut cybq_ctx, w: *const cybq_weight, x: *const c_void, xdt: c_int, M: i64,
                       y: *mut c_void, ydt: c_int, stream: *mut c_void) -> c_int;
    pub fn cybq_matmul_static(ctx: *mut cybq_ctx, w: *const cybq_weight, x: *const c_void, xdt: c_int, M: i64,
                              y: *mut c_void, ydt: c_int, stream: *mut c_void) -> c_int;
    pub fn cybq_set_prefill_mode(ctx: *mut cybq_ctx, mode: c_int) -> c_int;
    pub fn cybq_set_decode_mode(ctx: *mut cybq_ctx, mode: c_int) -> c_int;
    pub fn cybq_matmul_many(ctx: *mut cybq_ctx, count: i64, w: *const *const cybq_weight, x: *const *const c_void,
                            y: *const *mut c_void, xdt: c_int, M: i64, ydt: c_int, stream: *mut c_void) -> c_int;
    pub fn cybq_weight_fuse_pairs(ctx: *mut cybq_ctx, gate: *const cybq_weight, up: *const cybq_weight,
                                  out: *mut *mut cybq_weight) -> c_int;
    pub fn cybq_matmul_ex(ctx: *mut cybq_ctx, w: *const cybq_weight, x: *const c_void, xdt: c_int, M: i64,
                          y: *mut c_void, ydt: c_int, epilogue: c_int, residual: *const c_void,
                          stream: *mut c_void) -> c_int;
    pub fn cybq_matmul_norm(ctx: *mut cybq_ctx, w: *const cybq_weight, x: *const c_void, xdt: c_int, M: i64,
                            gamma: *const c_void, gdt: c_int, eps: c_float, y: *mut c_void, ydt: c_int,
                            epilogue: c_int, residual: *const c_void, stream: *mut c_void) -> c_int;
    pub fn cybq_matmul_many_ex(ctx: *mut cybq_ctx, count: i64, w: *const *const cybq_weight,
                               x: *const *const c_void, y: *const *mut c_void, epilogue: *const c_int,
                               residual: *const *const c_void, xdt: c_int, M: i64, ydt: c_int,
                               stream: *mut c_void) -> c_int;
    pub fn cybq_matmul_many_norm(ctx: *mut cybq_ctx, count: i64, w: *const *const cybq_weight,
                                 x: *const *const c_void, gamma: *const *const c_void, gdt: c_int, eps: c_float,
                                 y: *const *mut c_void, epilogue: *const c_int, residual: *const *const c_void,
                                 xdt: c_int, M: i64, ydt: c_int, stream: *mut c_void) -> c_int;
    pub fn cybq_dequant(ctx: *mut cybq_ctx, w: *const cybq_weight, out: *mut c_float, stream: *mut c_void) -> c_int;
    pub fn cybq_quantize(ctx: *mut cybq_ctx, quant: c_int, src: *const c_float, N: i64, K: i64, q_out: *mut c_void,
                         scales_out: *mut c_void, stream: *mut c_void) -> c_int;
    pub fn cybq_weight_from_device(ctx: *mut cybq_ctx, quant: c_int, N: i64, K: i64, q_dev: *const c_void,
                                   scales_dev: *const c_void, stream: *mut c_void,
                                   out: *mut *mut cybq_weight) -> c_int;
}
