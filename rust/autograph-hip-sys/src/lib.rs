//! Raw bindings to `libautograph_hip.so` (the C ABI of `include/autograph_hip.h`), one declaration
//! per entry point, in header order.  Status codes: 0 ok, negative argument errors (`AGH_E*`),
//! positive `hipError_t`.  This crate is source only: it has not been compiled (the image it was
//! written in has no Rust toolchain); `gen_bindings.py` writes this file from the header and
//! `tests/test_abi_cpu.py` checks every argument type against the header.
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_int, c_void};

pub const AGH_OK: c_int = 0;
pub const AGH_EINVAL: c_int = -1;
pub const AGH_ENOINIT: c_int = -2;
pub const AGH_ENULL: c_int = -3;
pub const AGH_ERANGE: c_int = -4;
pub const AGH_ACT_NONE: c_int = 0;
pub const AGH_ACT_RELU: c_int = 1;
pub const AGH_NOALLOC_SCRATCH_BYTES: usize = 16777216;

#[link(name = "autograph_hip")]
extern "C" {
    pub fn agh_init(device_index: c_int) -> c_int;
    pub fn agh_shutdown() -> c_int;
    pub fn agh_last_error_string() -> *const c_char;
    pub fn agh_device_info(name: *mut c_char, name_len: usize, compute_units: *mut c_int, total_mem_bytes: *mut usize) -> c_int;
    pub fn agh_malloc(ptr: *mut *mut c_void, bytes: usize) -> c_int;
    pub fn agh_free(ptr: *mut c_void) -> c_int;
    pub fn agh_cache_release() -> c_int;
    pub fn agh_cache_stats(cached_bytes: *mut usize, cached_blocks: *mut usize, live_blocks: *mut usize) -> c_int;
    pub fn agh_workspace_stats(workspace_bytes: *mut usize, retired_blocks: *mut usize) -> c_int;
    pub fn agh_memcpy_h2d(dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn agh_memcpy_d2h(dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn agh_memcpy_d2d(dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn agh_memset(dst: *mut c_void, byte_value: c_int, bytes: usize) -> c_int;
    pub fn agh_memcpy_d2h_async(dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn agh_host_alloc(ptr: *mut *mut c_void, bytes: usize) -> c_int;
    pub fn agh_host_free(ptr: *mut c_void) -> c_int;
    pub fn agh_sync() -> c_int;
    pub fn agh_stream() -> *mut c_void;
    pub fn agh_graph_begin() -> c_int;
    pub fn agh_graph_end(graph_exec: *mut *mut c_void) -> c_int;
    pub fn agh_graph_launch(graph_exec: *mut c_void) -> c_int;
    pub fn agh_graph_destroy(graph_exec: *mut c_void) -> c_int;
    pub fn agh_branch_begin() -> c_int;
    pub fn agh_branch_end() -> c_int;
    pub fn agh_branch_join() -> c_int;
    pub fn agh_event_create(event: *mut *mut c_void) -> c_int;
    pub fn agh_event_destroy(event: *mut c_void) -> c_int;
    pub fn agh_event_record(event: *mut c_void) -> c_int;
    pub fn agh_event_elapsed_ms(start: *mut c_void, stop: *mut c_void, ms: *mut f32) -> c_int;
    pub fn agh_gemm_f32(m: i64, k: i64, n: i64, alpha: f32, a: *const c_void, off_a: i64, rsa: i64, csa: i64, b: *const c_void, off_b: i64, rsb: i64, csb: i64, beta: f32, c: *mut c_void, off_c: i64, rsc: i64, csc: i64) -> c_int;
    pub fn agh_gemm_bf16(m: i64, k: i64, n: i64, alpha: f32, a: *const c_void, off_a: i64, rsa: i64, csa: i64, b: *const c_void, off_b: i64, rsb: i64, csb: i64, beta: f32, c: *mut c_void, off_c: i64, rsc: i64, csc: i64) -> c_int;
    pub fn agh_gemm_bf16_noalloc(m: i64, k: i64, n: i64, alpha: f32, a: *const c_void, off_a: i64, rsa: i64, csa: i64, b: *const c_void, off_b: i64, rsb: i64, csb: i64, beta: f32, c: *mut c_void, off_c: i64, rsc: i64, csc: i64) -> c_int;
    pub fn agh_gemm_f32_bias_act(m: i64, k: i64, n: i64, alpha: f32, a: *const c_void, off_a: i64, rsa: i64, csa: i64, b: *const c_void, off_b: i64, rsb: i64, csb: i64, beta: f32, c: *mut c_void, off_c: i64, rsc: i64, csc: i64, bias: *const c_void, off_bias: i64, bias_stride: i64, act: c_int) -> c_int;
    pub fn agh_gemm_bf16_bias_act(m: i64, k: i64, n: i64, alpha: f32, a: *const c_void, off_a: i64, rsa: i64, csa: i64, b: *const c_void, off_b: i64, rsb: i64, csb: i64, beta: f32, c: *mut c_void, off_c: i64, rsc: i64, csc: i64, bias: *const c_void, off_bias: i64, bias_stride: i64, act: c_int) -> c_int;
    pub fn agh_gemm_f32_batched(batch: i64, m: i64, k: i64, n: i64, alpha: f32, a: *const c_void, off_a: i64, rsa: i64, csa: i64, batch_stride_a: i64, b: *const c_void, off_b: i64, rsb: i64, csb: i64, batch_stride_b: i64, beta: f32, c: *mut c_void, off_c: i64, rsc: i64, csc: i64, batch_stride_c: i64, bias: *const c_void, off_bias: i64, bias_stride: i64, act: c_int) -> c_int;
    pub fn agh_gemm_bf16_batched(batch: i64, m: i64, k: i64, n: i64, alpha: f32, a: *const c_void, off_a: i64, rsa: i64, csa: i64, batch_stride_a: i64, b: *const c_void, off_b: i64, rsb: i64, csb: i64, batch_stride_b: i64, beta: f32, c: *mut c_void, off_c: i64, rsc: i64, csc: i64, batch_stride_c: i64, bias: *const c_void, off_bias: i64, bias_stride: i64, act: c_int) -> c_int;
    pub fn agh_im2col_conv2_f32(x: *const c_void, y: *mut c_void, bs: i64, c: i64, ih: i64, iw: i64, fh: i64, fw: i64, ph: i64, pw: i64, sh: i64, sw: i64, dh: i64, dw: i64) -> c_int;
    pub fn agh_im2col_conv2_bf16(x: *const c_void, y: *mut c_void, bs: i64, c: i64, ih: i64, iw: i64, fh: i64, fw: i64, ph: i64, pw: i64, sh: i64, sw: i64, dh: i64, dw: i64) -> c_int;
    pub fn agh_col2im_conv2_f32(x: *const c_void, y: *mut c_void, bs: i64, c: i64, ih: i64, iw: i64, fh: i64, fw: i64, ph: i64, pw: i64, sh: i64, sw: i64, dh: i64, dw: i64) -> c_int;
    pub fn agh_col2im_conv2_bf16(x: *const c_void, y: *mut c_void, bs: i64, c: i64, ih: i64, iw: i64, fh: i64, fw: i64, ph: i64, pw: i64, sh: i64, sw: i64, dh: i64, dw: i64) -> c_int;
    pub fn agh_conv2_backward_input_f32(dy: *const c_void, w: *const c_void, dx: *mut c_void, bs: i64, c: i64, ih: i64, iw: i64, oc: i64, fh: i64, fw: i64, ph: i64, pw: i64, sh: i64, sw: i64, dh: i64, dw: i64) -> c_int;
    pub fn agh_conv2_backward_input_bf16(dy: *const c_void, w: *const c_void, dx: *mut c_void, bs: i64, c: i64, ih: i64, iw: i64, oc: i64, fh: i64, fw: i64, ph: i64, pw: i64, sh: i64, sw: i64, dh: i64, dw: i64) -> c_int;
    pub fn agh_conv2_direct_f32(x: *const c_void, w: *const c_void, bias: *const c_void, y: *mut c_void, bs: i64, ic: i64, ih: i64, iw: i64, oc: i64, fh: i64, fw: i64, ph: i64, pw: i64, sh: i64, sw: i64, dh: i64, dw: i64, act: c_int, pool2x2: c_int) -> c_int;
    pub fn agh_conv2_direct_bf16(x: *const c_void, w: *const c_void, bias: *const c_void, y: *mut c_void, bs: i64, ic: i64, ih: i64, iw: i64, oc: i64, fh: i64, fw: i64, ph: i64, pw: i64, sh: i64, sw: i64, dh: i64, dw: i64, act: c_int, pool2x2: c_int) -> c_int;
    pub fn agh_lenet5_forward_f32(x: *const c_void, w1: *const c_void, w2: *const c_void, wd1: *const c_void, wd2: *const c_void, wd3: *const c_void, b3: *const c_void, logits: *mut c_void, bs: i64) -> c_int;
    pub fn agh_lenet5_forward_bf16(x: *const c_void, w1: *const c_void, w2: *const c_void, wd1: *const c_void, wd2: *const c_void, wd3: *const c_void, b3: *const c_void, logits: *mut c_void, bs: i64) -> c_int;
    pub fn agh_lenet5_forward_train_f32(x: *const c_void, w1: *const c_void, w2: *const c_void, wd1: *const c_void, wd2: *const c_void, wd3: *const c_void, b3: *const c_void, c1: *mut c_void, p1: *mut c_void, c2: *mut c_void, p2: *mut c_void, d1: *mut c_void, a1: *mut c_void, d2: *mut c_void, a2: *mut c_void, logits: *mut c_void, bs: i64) -> c_int;
    pub fn agh_lenet5_forward_train_bf16(x: *const c_void, w1: *const c_void, w2: *const c_void, wd1: *const c_void, wd2: *const c_void, wd3: *const c_void, b3: *const c_void, c1: *mut c_void, p1: *mut c_void, c2: *mut c_void, p2: *mut c_void, d1: *mut c_void, a1: *mut c_void, d2: *mut c_void, a2: *mut c_void, logits: *mut c_void, bs: i64) -> c_int;
    pub fn agh_lenet5_backward_f32(logits: *const c_void, target: *const c_void, dy: f32, c1: *const c_void, c2: *const c_void, d1: *const c_void, d2: *const c_void, w2: *const c_void, wd1: *const c_void, wd2: *const c_void, wd3: *const c_void, g_logits: *mut c_void, g_d2: *mut c_void, g_d1: *mut c_void, gm2: *mut c_void, gm1: *mut c_void, bs: i64) -> c_int;
    pub fn agh_lenet5_backward_bf16(logits: *const c_void, target: *const c_void, dy: f32, c1: *const c_void, c2: *const c_void, d1: *const c_void, d2: *const c_void, w2: *const c_void, wd1: *const c_void, wd2: *const c_void, wd3: *const c_void, g_logits: *mut c_void, g_d2: *mut c_void, g_d1: *mut c_void, gm2: *mut c_void, gm1: *mut c_void, bs: i64) -> c_int;
    pub fn agh_lenet5_dense_weight_grads_f32(a2: *const c_void, a1: *const c_void, f: *const c_void, g_logits: *const c_void, g_d2: *const c_void, g_d1: *const c_void, dwd3: *mut c_void, dwd2: *mut c_void, dwd1: *mut c_void, db3: *mut c_void, logits: *const c_void, target: *const c_void, loss: *mut c_void, bs: i64) -> c_int;
    pub fn agh_lenet5_dense_weight_grads_bf16(a2: *const c_void, a1: *const c_void, f: *const c_void, g_logits: *const c_void, g_d2: *const c_void, g_d1: *const c_void, dwd3: *mut c_void, dwd2: *mut c_void, dwd1: *mut c_void, db3: *mut c_void, logits: *const c_void, target: *const c_void, loss: *mut c_void, bs: i64) -> c_int;
    pub fn agh_lenet5_conv_weight_grads_f32(x: *const c_void, p1: *const c_void, gm1: *const c_void, gm2: *const c_void, dw1: *mut c_void, dw2: *mut c_void, bs: i64) -> c_int;
    pub fn agh_lenet5_conv_weight_grads_bf16(x: *const c_void, p1: *const c_void, gm1: *const c_void, gm2: *const c_void, dw1: *mut c_void, dw2: *mut c_void, bs: i64) -> c_int;
    pub fn agh_max_pool2_f32(x: *const c_void, y: *mut c_void, bc: i64, ih: i64, iw: i64, h: i64, w: i64, sh: i64, sw: i64) -> c_int;
    pub fn agh_max_pool2_bf16(x: *const c_void, y: *mut c_void, bc: i64, ih: i64, iw: i64, h: i64, w: i64, sh: i64, sw: i64) -> c_int;
    pub fn agh_max_pool2_backward_f32(dx_inout: *mut c_void, dy: *const c_void, bc: i64, ih: i64, iw: i64, h: i64, w: i64, sh: i64, sw: i64) -> c_int;
    pub fn agh_max_pool2_backward_bf16(dx_inout: *mut c_void, dy: *const c_void, bc: i64, ih: i64, iw: i64, h: i64, w: i64, sh: i64, sw: i64) -> c_int;
    pub fn agh_relu_max_pool2_f32(x: *const c_void, y: *mut c_void, bc: i64, ih: i64, iw: i64, h: i64, w: i64, sh: i64, sw: i64) -> c_int;
    pub fn agh_relu_max_pool2_bf16(x: *const c_void, y: *mut c_void, bc: i64, ih: i64, iw: i64, h: i64, w: i64, sh: i64, sw: i64) -> c_int;
    pub fn agh_max_pool2_relu_backward_f32(x: *const c_void, dy: *const c_void, dx: *mut c_void, bs: i64, c: i64, ih: i64, iw: i64, h: i64, w: i64, sh: i64, sw: i64, nhwc: c_int) -> c_int;
    pub fn agh_max_pool2_relu_backward_bf16(x: *const c_void, dy: *const c_void, dx: *mut c_void, bs: i64, c: i64, ih: i64, iw: i64, h: i64, w: i64, sh: i64, sw: i64, nhwc: c_int) -> c_int;
    pub fn agh_relu_f32(x: *const c_void, y: *mut c_void, n: i64) -> c_int;
    pub fn agh_relu_bf16(x: *const c_void, y: *mut c_void, n: i64) -> c_int;
    pub fn agh_relu_backward_f32(x: *const c_void, dy: *const c_void, dx: *mut c_void, n: i64) -> c_int;
    pub fn agh_relu_backward_bf16(x: *const c_void, dy: *const c_void, dx: *mut c_void, n: i64) -> c_int;
    pub fn agh_assign_f32(x: *const c_void, off_x: i64, sx0: i64, sx1: i64, sx2: i64, sx3: i64, y: *mut c_void, off_y: i64, sy0: i64, sy1: i64, sy2: i64, sy3: i64, d0: i64, d1: i64, d2: i64, d3: i64) -> c_int;
    pub fn agh_assign_bf16(x: *const c_void, off_x: i64, sx0: i64, sx1: i64, sx2: i64, sx3: i64, y: *mut c_void, off_y: i64, sy0: i64, sy1: i64, sy2: i64, sy3: i64, d0: i64, d1: i64, d2: i64, d3: i64) -> c_int;
    pub fn agh_scaled_add_f32(y: *mut c_void, alpha: f32, x: *const c_void, n: i64) -> c_int;
    pub fn agh_scaled_add_bf16(y: *mut c_void, alpha: f32, x: *const c_void, n: i64) -> c_int;
    pub fn agh_scaled_add_strided_f32(y: *mut c_void, off_y: i64, sy0: i64, sy1: i64, sy2: i64, sy3: i64, alpha: f32, x: *const c_void, off_x: i64, sx0: i64, sx1: i64, sx2: i64, sx3: i64, d0: i64, d1: i64, d2: i64, d3: i64) -> c_int;
    pub fn agh_scaled_add_strided_bf16(y: *mut c_void, off_y: i64, sy0: i64, sy1: i64, sy2: i64, sy3: i64, alpha: f32, x: *const c_void, off_x: i64, sx0: i64, sx1: i64, sx2: i64, sx3: i64, d0: i64, d1: i64, d2: i64, d3: i64) -> c_int;
    pub fn agh_sgd_momentum_f32(w: *mut c_void, dw: *const c_void, learning_rate: f32, momentum: f32, velocity: *mut c_void, n: i64) -> c_int;
    pub fn agh_sgd_momentum_bf16(w: *mut c_void, dw: *const c_void, learning_rate: f32, momentum: f32, velocity: *mut c_void, n: i64) -> c_int;
    pub fn agh_sum_axis0_f32(x: *const c_void, y: *mut c_void, rows: i64, cols: i64) -> c_int;
    pub fn agh_sum_axis0_bf16(x: *const c_void, y: *mut c_void, rows: i64, cols: i64) -> c_int;
    pub fn agh_cross_entropy_loss_f32(x: *const c_void, target_u8: *const c_void, bs: i64, classes: i64, loss: *mut f32) -> c_int;
    pub fn agh_cross_entropy_loss_bf16(x: *const c_void, target_u8: *const c_void, bs: i64, classes: i64, loss: *mut f32) -> c_int;
    pub fn agh_cross_entropy_backward_f32(x: *const c_void, target_u8: *const c_void, dy: f32, dx: *mut c_void, bs: i64, classes: i64) -> c_int;
    pub fn agh_cross_entropy_backward_bf16(x: *const c_void, target_u8: *const c_void, dy: f32, dx: *mut c_void, bs: i64, classes: i64) -> c_int;
    pub fn agh_accuracy_f32(x: *const c_void, target_u8: *const c_void, bs: i64, classes: i64, correct: *mut c_void) -> c_int;
    pub fn agh_accuracy_bf16(x: *const c_void, target_u8: *const c_void, bs: i64, classes: i64, correct: *mut c_void) -> c_int;
}
