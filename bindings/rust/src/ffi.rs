//! Raw declarations of the C ABI of libsliced_hip.so, one per function of `include/sliced_hip.h`
//! (same order, same argument names).  Every function returns a status: 0, a negative `SLHIP_E*`
//! code, or a positive hipError_t; `slhip_last_error_string` describes the last failure on the
//! calling thread.  Data pointers are device pointers of the context they are used with.
//!
//! `tests/test_rust_binding.py` of the library's tree checks that this file names exactly the
//! header's functions with the header's number of arguments.
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_void};

#[repr(C)]
pub struct SlhipCtx {
    _private: [u8; 0],
}
#[repr(C)]
pub struct SlhipEvent {
    _private: [u8; 0],
}
#[repr(C)]
pub struct SlhipGraph {
    _private: [u8; 0],
}

/// Status codes (`enum` of the header).
pub const SLHIP_OK: i32 = 0;
pub const SLHIP_EINVAL: i32 = -1;
pub const SLHIP_ENODEVICE: i32 = -2;
pub const SLHIP_EWORKSPACE: i32 = -3;
pub const SLHIP_EALIAS: i32 = -4;
pub const SLHIP_ECAPTURE: i32 = -5;

/// BinaryElementWise op codes (src/ops2/binary_ew/mod.rs:55-100 of the reference).
pub const SLHIP_ADD: i32 = 0;
pub const SLHIP_SUB: i32 = 1;
pub const SLHIP_MUL: i32 = 2;
pub const SLHIP_DIV: i32 = 3;

/// apply_fn / add_unary_grad op codes; `p`, `q` are the scalar parameters.
pub const SLHIP_SQUARE: i32 = 0;
pub const SLHIP_POW: i32 = 1;
pub const SLHIP_RELU: i32 = 2;
pub const SLHIP_EXP: i32 = 3;
pub const SLHIP_CLIP: i32 = 4;
pub const SLHIP_NEG_LN: i32 = 5;
pub const SLHIP_SCALE: i32 = 6;
pub const SLHIP_NEG_DIV: i32 = 7;
pub const SLHIP_TANH: i32 = 8;
pub const SLHIP_SIGMOID: i32 = 9;

pub const SLHIP_TAIL_AUTO: i32 = 0;
pub const SLHIP_TAIL_WHOLE: i32 = 1;
pub const SLHIP_TAIL_SPREAD: i32 = 2;
pub const SLHIP_TILE_AUTO: i32 = 0;
pub const SLHIP_TILE_128X128: i32 = 1;
pub const SLHIP_TILE_64X64: i32 = 3;
pub const SLHIP_TILE_128X128_WIDE: i32 = 4;

/// Elementwise programs (slhip_ew_program): limits, the unary marker or-ed into `op`, the flag
/// that stops the gradient at an instruction.
pub const SLHIP_EW_MAX_INPUTS: usize = 4;
pub const SLHIP_EW_MAX_OPS: usize = 8;
pub const SLHIP_EW_UNARY: u8 = 0x10;
pub const SLHIP_EW_NOGRAD: u8 = 0x1;

/// One instruction of an elementwise program: register j < 4 is input j, register 4 + i the
/// result of instruction i.
#[repr(C)]
#[derive(Clone, Copy, Debug, Default, PartialEq)]
pub struct SlhipEwInsn {
    pub op: u8,
    pub src0: u8,
    pub src1: u8,
    pub flags: u8,
    pub p: f32,
    pub q: f32,
}

extern "C" {
    pub fn slhip_init(device_ordinal: i32, ctx: *mut *mut SlhipCtx) -> i32;
    pub fn slhip_init_on_stream(device_ordinal: i32, hip_stream: *mut c_void, ctx: *mut *mut SlhipCtx) -> i32;
    pub fn slhip_destroy(ctx: *mut SlhipCtx) -> i32;
    pub fn slhip_last_error_string() -> *const c_char;
    pub fn slhip_device_name(ctx: *mut SlhipCtx, buf: *mut c_char, buflen: usize) -> i32;
    pub fn slhip_stream(ctx: *mut SlhipCtx, hip_stream: *mut *mut c_void) -> i32;
    pub fn slhip_workspace_bytes(ctx: *mut SlhipCtx) -> usize;
    pub fn slhip_workspace(ctx: *mut SlhipCtx, dptr: *mut *mut c_void) -> i32;
    pub fn slhip_malloc(ctx: *mut SlhipCtx, bytes: usize, dptr: *mut *mut c_void) -> i32;
    pub fn slhip_free(ctx: *mut SlhipCtx, dptr: *mut c_void) -> i32;
    pub fn slhip_memcpy_h2d(ctx: *mut SlhipCtx, dst_dev: *mut c_void, src_host: *const c_void, bytes: usize) -> i32;
    pub fn slhip_memcpy_d2h(ctx: *mut SlhipCtx, dst_host: *mut c_void, src_dev: *const c_void, bytes: usize) -> i32;
    pub fn slhip_memcpy_d2d(ctx: *mut SlhipCtx, dst_dev: *mut c_void, src_dev: *const c_void, bytes: usize) -> i32;
    pub fn slhip_memset(ctx: *mut SlhipCtx, dptr: *mut c_void, byte_value: i32, bytes: usize) -> i32;
    pub fn slhip_fill(ctx: *mut SlhipCtx, n: usize, value: f32, x: *mut f32) -> i32;
    pub fn slhip_sync(ctx: *mut SlhipCtx) -> i32;
    pub fn slhip_event_create(ctx: *mut SlhipCtx, ev: *mut *mut SlhipEvent) -> i32;
    pub fn slhip_event_record(ctx: *mut SlhipCtx, ev: *mut SlhipEvent) -> i32;
    pub fn slhip_event_elapsed_ms(start: *mut SlhipEvent, stop: *mut SlhipEvent, ms: *mut f32) -> i32;
    pub fn slhip_event_destroy(ev: *mut SlhipEvent) -> i32;
    pub fn slhip_graph_begin(ctx: *mut SlhipCtx) -> i32;
    pub fn slhip_graph_end(ctx: *mut SlhipCtx, graph: *mut *mut SlhipGraph) -> i32;
    pub fn slhip_graph_launch(ctx: *mut SlhipCtx, graph: *mut SlhipGraph) -> i32;
    pub fn slhip_graph_node_count(graph: *mut SlhipGraph, nodes: *mut usize) -> i32;
    pub fn slhip_graph_destroy(graph: *mut SlhipGraph) -> i32;
    pub fn slhip_rand_uniform(
        ctx: *mut SlhipCtx,
        seed: u64,
        tag: u64,
        lo: f32,
        hi: f32,
        n: usize,
        x: *mut f32,
    ) -> i32;
    pub fn slhip_sgemm(
        ctx: *mut SlhipCtx,
        trans_a: i32,
        trans_b: i32,
        m: usize,
        n: usize,
        k: usize,
        a: *const f32,
        b: *const f32,
        c: *mut f32,
        beta: f32,
    ) -> i32;
    pub fn slhip_sgemm_relu_mask(
        ctx: *mut SlhipCtx,
        trans_a: i32,
        trans_b: i32,
        m: usize,
        n: usize,
        k: usize,
        a: *const f32,
        b: *const f32,
        pre: *const f32,
        c: *mut f32,
        beta: f32,
    ) -> i32;
    pub fn slhip_gemm_tail_policy(ctx: *mut SlhipCtx, policy: i32) -> i32;
    pub fn slhip_gemm_tile_policy(ctx: *mut SlhipCtx, policy: i32) -> i32;
    pub fn slhip_gemm_plan_describe(ctx: *mut SlhipCtx, buf: *mut c_char, len: usize) -> i32;
    pub fn slhip_gemm(
        ctx: *mut SlhipCtx,
        m: usize,
        k: usize,
        n: usize,
        lhs: *const f32,
        rhs: *const f32,
        out: *mut f32,
    ) -> i32;
    pub fn slhip_gemm_grad(
        ctx: *mut SlhipCtx,
        m: usize,
        k: usize,
        n: usize,
        lhs: *const f32,
        rhs: *const f32,
        lhs_grad: *mut f32,
        rhs_grad: *mut f32,
        out_grad: *const f32,
        beta: f32,
    ) -> i32;
    pub fn slhip_linear_fwd(
        ctx: *mut SlhipCtx,
        m: usize,
        k: usize,
        n: usize,
        x: *const f32,
        w: *const f32,
        bias: *const f32,
        relu: i32,
        pre_act: *mut f32,
        out: *mut f32,
    ) -> i32;
    pub fn slhip_linear_grad(
        ctx: *mut SlhipCtx,
        m: usize,
        k: usize,
        n: usize,
        x: *const f32,
        w: *const f32,
        x_grad: *mut f32,
        relu_pre: *const f32,
        w_grad: *mut f32,
        bias_grad: *mut f32,
        out_grad: *const f32,
        beta: f32,
    ) -> i32;
    pub fn slhip_sum_rows(ctx: *mut SlhipCtx, rows: usize, cols: usize, x: *const f32, out: *mut f32) -> i32;
    pub fn slhip_sum_cols(ctx: *mut SlhipCtx, rows: usize, cols: usize, x: *const f32, out: *mut f32) -> i32;
    pub fn slhip_max_rows(ctx: *mut SlhipCtx, rows: usize, cols: usize, x: *const f32, out: *mut f32) -> i32;
    pub fn slhip_max_cols(ctx: *mut SlhipCtx, rows: usize, cols: usize, x: *const f32, out: *mut f32) -> i32;
    pub fn slhip_mean_rows(ctx: *mut SlhipCtx, rows: usize, cols: usize, x: *const f32, out: *mut f32) -> i32;
    pub fn slhip_mean_cols(ctx: *mut SlhipCtx, rows: usize, cols: usize, x: *const f32, out: *mut f32) -> i32;
    pub fn slhip_sum_rows_static(ctx: *mut SlhipCtx, rows: usize, cols: usize, x: *const f32, out: *mut f32) -> i32;
    pub fn slhip_sum(ctx: *mut SlhipCtx, len: usize, x: *const f32, out_dev: *mut f32) -> i32;
    pub fn slhip_max(ctx: *mut SlhipCtx, len: usize, x: *const f32, out_dev: *mut f32) -> i32;
    pub fn slhip_mean(ctx: *mut SlhipCtx, len: usize, x: *const f32, out_dev: *mut f32) -> i32;
    pub fn slhip_sum_rows_grad(
        ctx: *mut SlhipCtx,
        rows: usize,
        cols: usize,
        x_grad: *mut f32,
        out_grad: *const f32,
    ) -> i32;
    pub fn slhip_sum_cols_grad(
        ctx: *mut SlhipCtx,
        rows: usize,
        cols: usize,
        x_grad: *mut f32,
        out_grad: *const f32,
    ) -> i32;
    pub fn slhip_max_rows_grad(
        ctx: *mut SlhipCtx,
        rows: usize,
        cols: usize,
        out: *const f32,
        x: *const f32,
        x_grad: *mut f32,
        out_grad: *const f32,
    ) -> i32;
    pub fn slhip_max_cols_grad(
        ctx: *mut SlhipCtx,
        rows: usize,
        cols: usize,
        out: *const f32,
        x: *const f32,
        x_grad: *mut f32,
        out_grad: *const f32,
    ) -> i32;
    pub fn slhip_mean_rows_grad(
        ctx: *mut SlhipCtx,
        rows: usize,
        cols: usize,
        x_grad: *mut f32,
        out_grad: *const f32,
    ) -> i32;
    pub fn slhip_mean_cols_grad(
        ctx: *mut SlhipCtx,
        rows: usize,
        cols: usize,
        x_grad: *mut f32,
        out_grad: *const f32,
    ) -> i32;
    pub fn slhip_softmax(ctx: *mut SlhipCtx, samples: usize, features: usize, x: *const f32, out: *mut f32) -> i32;
    pub fn slhip_softmax_grad(
        ctx: *mut SlhipCtx,
        samples: usize,
        features: usize,
        x_grad: *mut f32,
        out: *const f32,
        out_grad: *const f32,
        beta: f32,
    ) -> i32;
    pub fn slhip_transpose(
        ctx: *mut SlhipCtx,
        rows: usize,
        cols: usize,
        x: *const f32,
        out: *mut f32,
        beta: f32,
    ) -> i32;
    pub fn slhip_add_row(
        ctx: *mut SlhipCtx,
        rows: usize,
        cols: usize,
        lhs: *const f32,
        rhs: *const f32,
        out: *mut f32,
    ) -> i32;
    pub fn slhip_add_row_grad(
        ctx: *mut SlhipCtx,
        rows: usize,
        cols: usize,
        lhs_grad: *mut f32,
        rhs_grad: *mut f32,
        out_grad: *const f32,
    ) -> i32;
    pub fn slhip_add_row_mut_grad(
        ctx: *mut SlhipCtx,
        rows: usize,
        cols: usize,
        rhs_grad: *mut f32,
        out_grad: *const f32,
    ) -> i32;
    pub fn slhip_row_op(
        ctx: *mut SlhipCtx,
        op: i32,
        rows: usize,
        cols: usize,
        lhs: *const f32,
        rhs: *const f32,
        out: *mut f32,
    ) -> i32;
    pub fn slhip_row_op_grad(
        ctx: *mut SlhipCtx,
        op: i32,
        rows: usize,
        cols: usize,
        lhs: *const f32,
        rhs: *const f32,
        lhs_grad: *mut f32,
        rhs_grad: *mut f32,
        out_grad: *const f32,
    ) -> i32;
    pub fn slhip_col_op(
        ctx: *mut SlhipCtx,
        op: i32,
        rows: usize,
        cols: usize,
        lhs: *const f32,
        rhs: *const f32,
        out: *mut f32,
    ) -> i32;
    pub fn slhip_col_op_grad(
        ctx: *mut SlhipCtx,
        op: i32,
        rows: usize,
        cols: usize,
        lhs: *const f32,
        rhs: *const f32,
        lhs_grad: *mut f32,
        rhs_grad: *mut f32,
        out_grad: *const f32,
    ) -> i32;
    pub fn slhip_ew_binary(ctx: *mut SlhipCtx, op: i32, n: usize, l: *const f32, r: *const f32, out: *mut f32) -> i32;
    pub fn slhip_ew_binary_grad(
        ctx: *mut SlhipCtx,
        op: i32,
        n: usize,
        l: *const f32,
        r: *const f32,
        lg: *mut f32,
        rg: *mut f32,
        g: *const f32,
    ) -> i32;
    pub fn slhip_ew_unary(ctx: *mut SlhipCtx, op: i32, p: f32, q: f32, n: usize, x: *const f32, out: *mut f32) -> i32;
    pub fn slhip_ew_unary_grad(
        ctx: *mut SlhipCtx,
        op: i32,
        p: f32,
        n: usize,
        x: *const f32,
        x_grad: *mut f32,
        out_grad: *const f32,
    ) -> i32;
    pub fn slhip_ew_chain(
        ctx: *mut SlhipCtx,
        n: usize,
        a: *const f32,
        b: *const f32,
        c: *const f32,
        d: *const f32,
        out: *mut f32,
    ) -> i32;
    pub fn slhip_ew_program(
        ctx: *mut SlhipCtx,
        n: usize,
        n_inputs: usize,
        inputs: *const *const f32,
        n_ops: usize,
        prog: *const SlhipEwInsn,
        out: *mut f32,
    ) -> i32;
    pub fn slhip_ew_program_grad(
        ctx: *mut SlhipCtx,
        n: usize,
        n_inputs: usize,
        inputs: *const *const f32,
        input_grads: *const *mut f32,
        n_ops: usize,
        prog: *const SlhipEwInsn,
        out_grad: *const f32,
    ) -> i32;
    pub fn slhip_sgd_step(ctx: *mut SlhipCtx, n: usize, p: *mut f32, g: *const f32, lr: f32) -> i32;
    pub fn slhip_mlp3_mse_step(ctx: *mut SlhipCtx, batch: usize, d_in: usize, d_h: usize, d_out: usize, x: *const f32,
                               target: *const f32, w1: *mut f32, b1: *mut f32, w2: *mut f32, b2: *mut f32, w3: *mut f32, b3: *mut f32,
                               grads: *const *mut f32, lr: f32, loss_dev: *mut f32) -> i32;
    pub fn slhip_sgd_step_multi(
        ctx: *mut SlhipCtx,
        count: usize,
        params: *const *mut f32,
        grads: *const *const f32,
        lens: *const usize,
        lr: f32,
    ) -> i32;
    pub fn slhip_cce(
        ctx: *mut SlhipCtx,
        rows: usize,
        cols: usize,
        preds: *const f32,
        targets: *const f32,
        loss: *mut f32,
    ) -> i32;
    pub fn slhip_cce_grad(
        ctx: *mut SlhipCtx,
        rows: usize,
        cols: usize,
        preds: *const f32,
        targets: *const f32,
        grad: *mut f32,
    ) -> i32;
    pub fn slhip_onehot(ctx: *mut SlhipCtx, n: usize, classes: usize, cls: *const f32, out: *mut f32) -> i32;
    pub fn slhip_linear_fwd_bits(
        ctx: *mut SlhipCtx,
        m: usize,
        k: usize,
        n: usize,
        x: *const f32,
        w: *const f32,
        bias: *const f32,
        bits: *mut u32,
        out: *mut f32,
    ) -> i32;
    pub fn slhip_sgemm_relu_bits(
        ctx: *mut SlhipCtx,
        trans_a: i32,
        trans_b: i32,
        m: usize,
        n: usize,
        k: usize,
        a: *const f32,
        b: *const f32,
        bits: *const u32,
        c: *mut f32,
        beta: f32,
    ) -> i32;
    pub fn slhip_relu_grad_bits(
        ctx: *mut SlhipCtx,
        rows: usize,
        cols: usize,
        bits: *const u32,
        x_grad: *mut f32,
        out_grad: *const f32,
    ) -> i32;
    pub fn slhip_mse(ctx: *mut SlhipCtx, n: usize, x: *const f32, y: *const f32, loss_dev: *mut f32) -> i32;
    pub fn slhip_mse_grad(
        ctx: *mut SlhipCtx,
        n: usize,
        x: *const f32,
        y: *const f32,
        x_grad: *mut f32,
        upstream_dev: *const f32,
    ) -> i32;
    pub fn slhip_softmax_cce(
        ctx: *mut SlhipCtx,
        rows: usize,
        cols: usize,
        logits: *const f32,
        targets: *const f32,
        probs: *mut f32,
        loss_rows: *mut f32,
    ) -> i32;
    pub fn slhip_softmax_cce_grad(
        ctx: *mut SlhipCtx,
        rows: usize,
        cols: usize,
        probs: *const f32,
        targets: *const f32,
        logits_grad: *mut f32,
        beta: f32,
        upstream_dev: *const f32,
    ) -> i32;
    pub fn slhip_onehot_grad(
        ctx: *mut SlhipCtx,
        n: usize,
        classes: usize,
        cls: *const f32,
        cls_grad: *mut f32,
        out_grad: *const f32,
    ) -> i32;
    pub fn slhip_diagflat(ctx: *mut SlhipCtx, n: usize, x: *const f32, out: *mut f32) -> i32;
    pub fn slhip_diagflat_grad(ctx: *mut SlhipCtx, n: usize, x_grad: *mut f32, out_grad: *const f32) -> i32;
}
