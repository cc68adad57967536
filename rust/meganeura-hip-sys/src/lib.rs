//! Raw FFI bindings to `libmgn_hip.so`, the MI355X (gfx950) backend for meganeura's quantized
//! (Q4 / Q8) matmul path.  One `extern "C"` declaration per symbol of `include/mgn_hip.h`,
//! `include/mgn_bench.h` (module `bench`) and `include/mgn_session.h` (module `session`);
//! `tests/test_rust_binding.py` holds the three in step (names, arity, argument types).
//!
//! Written against the headers and never compiled here: the build image has no Rust toolchain.
//! `src/runtime.rs` of meganeura calls these in place of its blade-graphics dispatch for
//! dispatches whose `weight_format` is Q4 / Q8 (`Session::set_parameter`, runtime.rs:2327-2345;
//! `Session::step` / `bind_dispatch`, runtime.rs:2843-2959, 3073-3122).
#![allow(non_camel_case_types)]
use std::os::raw::{c_char, c_int, c_void};

#[repr(C)]
pub struct mgn_ctx {
    _private: [u8; 0],
}
#[repr(C)]
pub struct mgn_buf {
    _private: [u8; 0],
}
#[repr(C)]
pub struct mgn_weight {
    _private: [u8; 0],
}

/// `mgn_status`: 0 is `MGN_OK`; the message of a failed call is `mgn_last_error(ctx)`.
pub type mgn_status = c_int;
pub const MGN_OK: mgn_status = 0;
pub const MGN_EINVAL: mgn_status = 1;
pub const MGN_ENOMEM: mgn_status = 2;
pub const MGN_EHIP: mgn_status = 3;
pub const MGN_ENOTFOUND: mgn_status = 4;
pub const MGN_ENODEVICE: mgn_status = 5;
pub const MGN_EUNSUPPORTED: mgn_status = 6;
pub const MGN_ERANGE: mgn_status = 7;
pub const MGN_ETIMEOUT: mgn_status = 8;

/// `mgn_fmt` = `compile::WeightFormat::{Q4, Q8}` (src/compile.rs:8-29).
pub type mgn_fmt = c_int;
pub const MGN_FMT_Q4: mgn_fmt = 0;
pub const MGN_FMT_Q8: mgn_fmt = 1;

pub type mgn_act_range = c_int;
pub const MGN_ACT_ANY: mgn_act_range = 0;
pub const MGN_ACT_FP16_RANGE: mgn_act_range = 1;

/// `mgn_route`: kernel family; a runtime leaves it at `MGN_ROUTE_AUTO`.
pub type mgn_route = c_int;
pub const MGN_ROUTE_AUTO: mgn_route = 0;
pub const MGN_ROUTE_GENERIC: mgn_route = 1;
pub const MGN_ROUTE_GEMV_VALU: mgn_route = 2;
pub const MGN_ROUTE_GEMV_MFMA: mgn_route = 3;
pub const MGN_ROUTE_GEMM_MFMA: mgn_route = 4;
pub const MGN_ROUTE_TILE_MFMA: mgn_route = 5;

/// `mgn_unary`: the operations `fuse_epilogues` folds into a matmul (src/compile.rs:915-1035).
pub type mgn_unary = c_int;
pub const MGN_UNARY_NONE: mgn_unary = 0;
pub const MGN_UNARY_RELU: mgn_unary = 1;
pub const MGN_UNARY_SIGMOID: mgn_unary = 2;
pub const MGN_UNARY_NEG: mgn_unary = 3;
pub const MGN_UNARY_SILU: mgn_unary = 4;

/// `mgn_prologue`: what the activations of a decode matmul go through while they are staged.
pub type mgn_prologue = c_int;
pub const MGN_PROLOGUE_NONE: mgn_prologue = 0;
pub const MGN_PROLOGUE_RMS_NORM: mgn_prologue = 1;
pub const MGN_PROLOGUE_SWIGLU: mgn_prologue = 2;

/// Bytes of split-K partial sums `mgn_matmul_q_static` can hold (`MGN_STATIC_WORKSPACE_BYTES`).
pub const MGN_STATIC_WORKSPACE_BYTES: usize = 4 << 20;

#[repr(C)]
#[derive(Clone, Copy)]
pub struct mgn_matmul_item {
    pub w: *const mgn_weight,
    pub d: *const mgn_buf,
    pub c: *mut mgn_buf,
}

/// A chain of dependent one-row matmuls served by one launch (`mgn_chain_create`).
#[repr(C)]
pub struct mgn_chain {
    _private: [u8; 0],
}

/// One stage of a chain: `C = f(prologue(A) x W + D)`.
#[repr(C)]
#[derive(Clone, Copy)]
pub struct mgn_chain_stage {
    pub w: *const mgn_weight,
    pub a: *const mgn_buf,
    pub prologue: mgn_prologue,
    pub norm_weight: *const mgn_buf,
    pub eps: f32,
    pub d: *const mgn_buf,
    pub c: *mut mgn_buf,
    pub ops: *const mgn_unary,
    pub n_ops: usize,
}

#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct mgn_plan_info {
    pub route: c_int,
    pub grid: [u32; 3],
    pub threads: u32,
    pub lds_bytes: u32,
    pub waves_n: u32,
    pub k_splits: u32,
    pub k_parts: u32,
    pub steps: u32,
    pub quads_per_wave: u32,
    pub full_steps: u32,
    pub tail_blocks: u32,
    pub workspace_bytes: u64,
}

#[link(name = "mgn_hip")]
extern "C" {
    pub fn mgn_ctx_create(device_id: c_int, out: *mut *mut mgn_ctx) -> mgn_status;
    pub fn mgn_ctx_destroy(ctx: *mut mgn_ctx);
    pub fn mgn_last_error(ctx: *const mgn_ctx) -> *const c_char;
    pub fn mgn_sync(ctx: *mut mgn_ctx) -> mgn_status;
    pub fn mgn_ctx_set_activation_range(ctx: *mut mgn_ctx, range: mgn_act_range) -> mgn_status;
    pub fn mgn_ctx_set_shared_device(ctx: *mut mgn_ctx, shared: c_int) -> mgn_status;
    pub fn mgn_buf_alloc(ctx: *mut mgn_ctx, bytes: usize, out: *mut *mut mgn_buf) -> mgn_status;
    pub fn mgn_buf_free(ctx: *mut mgn_ctx, buf: *mut mgn_buf);
    pub fn mgn_buf_size(buf: *const mgn_buf) -> usize;
    pub fn mgn_buf_device_ptr(buf: *const mgn_buf) -> *mut c_void;
    pub fn mgn_buf_upload(ctx: *mut mgn_ctx, buf: *mut mgn_buf, offset: usize, src: *const c_void, bytes: usize) -> mgn_status;
    pub fn mgn_buf_download(ctx: *mut mgn_ctx, buf: *const mgn_buf, offset: usize, dst: *mut c_void, bytes: usize) -> mgn_status;
    pub fn mgn_buf_copy(ctx: *mut mgn_ctx, dst: *mut mgn_buf, src: *const mgn_buf, bytes: usize) -> mgn_status;
    pub fn mgn_packed_size(fmt: mgn_fmt, rows: usize, cols: usize) -> usize;
    pub fn mgn_quantize_ref(fmt: mgn_fmt, w: *const f32, rows: usize, cols: usize, out: *mut u8) -> mgn_status;
    pub fn mgn_dequantize_ref(fmt: mgn_fmt, input: *const u8, rows: usize, cols: usize, out: *mut f32) -> mgn_status;
    pub fn mgn_weight_create(ctx: *mut mgn_ctx, fmt: mgn_fmt, w: *const f32, rows: usize, cols: usize, out: *mut *mut mgn_weight) -> mgn_status;
    pub fn mgn_weight_create_packed(ctx: *mut mgn_ctx, fmt: mgn_fmt, packed: *const u8, rows: usize, cols: usize, out: *mut *mut mgn_weight) -> mgn_status;
    pub fn mgn_quantize_ref_nk(fmt: mgn_fmt, w_nk: *const f32, n_rows: usize, k_cols: usize, out: *mut u8) -> mgn_status;
    pub fn mgn_weight_create_nk(ctx: *mut mgn_ctx, fmt: mgn_fmt, w_nk: *const f32, n_rows: usize, k_cols: usize, out: *mut *mut mgn_weight) -> mgn_status;
    pub fn mgn_weight_create_device(ctx: *mut mgn_ctx, fmt: mgn_fmt, w_f32: *const mgn_buf, rows: usize, cols: usize, out: *mut *mut mgn_weight) -> mgn_status;
    pub fn mgn_weight_free(ctx: *mut mgn_ctx, w: *mut mgn_weight);
    pub fn mgn_weight_info(w: *const mgn_weight, fmt: *mut mgn_fmt, rows: *mut usize, cols: *mut usize) -> mgn_status;
    pub fn mgn_weight_dequantize(ctx: *mut mgn_ctx, w: *const mgn_weight, out_host: *mut f32) -> mgn_status;
    pub fn mgn_weight_export_ref(ctx: *mut mgn_ctx, w: *const mgn_weight, out_packed: *mut u8) -> mgn_status;
    pub fn mgn_weight_save(ctx: *mut mgn_ctx, w: *const mgn_weight, path: *const c_char) -> mgn_status;
    pub fn mgn_weight_load(ctx: *mut mgn_ctx, path: *const c_char, out: *mut *mut mgn_weight) -> mgn_status;
    pub fn mgn_matmul_q(ctx: *mut mgn_ctx, a: *const mgn_buf, w: *const mgn_weight, d: *const mgn_buf, c: *mut mgn_buf, m: u32) -> mgn_status;
    pub fn mgn_matmul_q_f16a(ctx: *mut mgn_ctx, a_f16: *const mgn_buf, w: *const mgn_weight, d: *const mgn_buf, c: *mut mgn_buf, m: u32) -> mgn_status;
    pub fn mgn_matmul_q_static(ctx: *mut mgn_ctx, a: *const mgn_buf, w: *const mgn_weight, d: *const mgn_buf, c: *mut mgn_buf, m: u32) -> mgn_status;
    pub fn mgn_matmul_q_epilogue(ctx: *mut mgn_ctx, a: *const mgn_buf, w: *const mgn_weight, d: *const mgn_buf, c: *mut mgn_buf, m: u32, ops: *const mgn_unary, n_ops: usize) -> mgn_status;
    pub fn mgn_matmul_q_at(ctx: *mut mgn_ctx, a_t: *const mgn_buf, w: *const mgn_weight, d: *const mgn_buf, c: *mut mgn_buf, m: u32, ops: *const mgn_unary, n_ops: usize) -> mgn_status;
    pub fn mgn_matmul_q_plan(fmt: mgn_fmt, m: u32, k: u64, n: u64, a_is_f16: c_int, num_cus: c_int, out: *mut mgn_plan_info) -> mgn_status;
    pub fn mgn_matmul_q_rms_norm(ctx: *mut mgn_ctx, x: *const mgn_buf, norm_weight: *const mgn_buf, eps: f32, w: *const mgn_weight, d: *const mgn_buf, c: *mut mgn_buf, m: u32) -> mgn_status;
    pub fn mgn_matmul_q_swiglu(ctx: *mut mgn_ctx, gate_up: *const mgn_buf, w: *const mgn_weight, d: *const mgn_buf, c: *mut mgn_buf, m: u32) -> mgn_status;
    pub fn mgn_matmul_q_can_fuse(ctx: *mut mgn_ctx, w: *const mgn_weight, m: u32) -> c_int;
    pub fn mgn_matmul_q_batch(ctx: *mut mgn_ctx, a: *const mgn_buf, prologue: mgn_prologue, norm_weight: *const mgn_buf, eps: f32, items: *const mgn_matmul_item, count: usize, m: u32) -> mgn_status;
    pub fn mgn_chain_create(ctx: *mut mgn_ctx, stages: *const mgn_chain_stage, count: usize, m: u32, out: *mut *mut mgn_chain) -> mgn_status;
    pub fn mgn_chain_run(ctx: *mut mgn_ctx, chain: *mut mgn_chain) -> mgn_status;
    pub fn mgn_chain_free(ctx: *mut mgn_ctx, chain: *mut mgn_chain);
    pub fn mgn_timer_start(ctx: *mut mgn_ctx) -> mgn_status;
    pub fn mgn_timer_stop(ctx: *mut mgn_ctx, elapsed_ms: *mut f32) -> mgn_status;
    pub fn mgn_version() -> *const c_char;
    pub fn mgn_built_for() -> *const c_char;
}

/// `include/mgn_bench.h`: entry points only test and benchmark harnesses use.
pub mod bench {
    use super::*;

    #[link(name = "mgn_hip")]
    extern "C" {
        pub fn mgn_ctx_set_route(ctx: *mut mgn_ctx, route: mgn_route) -> mgn_status;
        pub fn mgn_ctx_set_spin_limit(ctx: *mut mgn_ctx, polls: u32) -> mgn_status;
        pub fn mgn_engine_clock_mhz(ctx: *mut mgn_ctx, loaded: c_int, mhz: *mut f32, cycles_per_round: *mut f32) -> mgn_status;
        pub fn mgn_matmul_q_loop(ctx: *mut mgn_ctx, a: *const mgn_buf, a_is_f16: c_int, weights: *const *const mgn_weight, count: usize, d: *const mgn_buf, c: *mut mgn_buf, m: u32, steps: u32) -> mgn_status;
        pub fn mgn_weight_read_loop(ctx: *mut mgn_ctx, weights: *const *const mgn_weight, count: usize, steps: u32, pattern: c_int) -> mgn_status;
    }
}

/// `include/mgn_session.h`: the Graph / Session mirror (C++ inside the library), for hosts that
/// want the whole `build_inference_session` flow rather than the per-dispatch calls.
pub mod session {
    use super::*;

    #[repr(C)]
    pub struct mgn_graph {
        _private: [u8; 0],
    }
    #[repr(C)]
    pub struct mgn_session {
        _private: [u8; 0],
    }

    /// `mgn_shader` = the `compile::ShaderEntry` values that can appear in a plan here.
    pub type mgn_shader = i32;
    pub const MGN_SHADER_MATMUL: mgn_shader = 0;
    pub const MGN_SHADER_MATMUL_GEMV: mgn_shader = 1;
    pub const MGN_SHADER_FUSED_MATMUL_ADD: mgn_shader = 2;
    pub const MGN_SHADER_MATMUL_GEMV_ADD: mgn_shader = 3;
    pub const MGN_SHADER_ADD: mgn_shader = 4;
    pub const MGN_SHADER_SWIGLU: mgn_shader = 5;
    pub const MGN_SHADER_SWIGLU_CONCAT: mgn_shader = 6;
    pub const MGN_SHADER_RMS_NORM: mgn_shader = 7;
    pub const MGN_SHADER_MATMUL_BT: mgn_shader = 8;
    pub const MGN_SHADER_MATMUL_GEMV_BT: mgn_shader = 9;
    pub const MGN_SHADER_RELU: mgn_shader = 10;
    pub const MGN_SHADER_SIGMOID: mgn_shader = 11;
    pub const MGN_SHADER_NEG: mgn_shader = 12;
    pub const MGN_SHADER_SILU: mgn_shader = 13;
    pub const MGN_SHADER_MATMUL_AT: mgn_shader = 14;
    pub const MGN_SHADER_FUSED_MATMUL_AT_ADD: mgn_shader = 15;
    pub const MGN_SHADER_FUSED_MATMUL_BT_ADD: mgn_shader = 16;

    /// `compile::Dispatch` (src/compile.rs:435-488), the fields this path uses.
    #[repr(C)]
    #[derive(Clone, Copy, Debug, Default)]
    pub struct mgn_dispatch_info {
        pub shader: i32,
        pub workgroups: [u32; 3],
        pub params: [u32; 4],
        pub weight_format: i32,
        pub epilogue: u32,
    }

    #[link(name = "mgn_hip")]
    extern "C" {
        pub fn mgn_graph_new() -> *mut mgn_graph;
        pub fn mgn_graph_free(g: *mut mgn_graph);
        pub fn mgn_graph_last_error(g: *const mgn_graph) -> *const c_char;
        pub fn mgn_graph_input(g: *mut mgn_graph, name: *const c_char, rows: usize, cols: usize) -> i32;
        pub fn mgn_graph_parameter(g: *mut mgn_graph, name: *const c_char, rows: usize, cols: usize) -> i32;
        pub fn mgn_graph_parameter_q4(g: *mut mgn_graph, name: *const c_char, rows: usize, cols: usize) -> i32;
        pub fn mgn_graph_parameter_q8(g: *mut mgn_graph, name: *const c_char, rows: usize, cols: usize) -> i32;
        pub fn mgn_graph_matmul(g: *mut mgn_graph, a: i32, b: i32) -> i32;
        pub fn mgn_graph_matmul_bt(g: *mut mgn_graph, a: i32, b: i32) -> i32;
        pub fn mgn_graph_matmul_at(g: *mut mgn_graph, a: i32, b: i32) -> i32;
        pub fn mgn_graph_add(g: *mut mgn_graph, a: i32, b: i32) -> i32;
        pub fn mgn_graph_swiglu(g: *mut mgn_graph, gate: i32, up: i32) -> i32;
        pub fn mgn_graph_rms_norm(g: *mut mgn_graph, x: i32, weight: i32, eps: f32) -> i32;
        pub fn mgn_graph_unary(g: *mut mgn_graph, kind: i32, x: i32) -> i32;
        pub fn mgn_graph_set_outputs(g: *mut mgn_graph, ids: *const i32, count: usize) -> mgn_status;
        pub fn mgn_graph_compile(g: *const mgn_graph, out: *mut mgn_dispatch_info, cap: usize, count: *mut usize) -> mgn_status;
        pub fn mgn_build_inference_session(g: *const mgn_graph, device_id: c_int, out: *mut *mut mgn_session) -> mgn_status;
        pub fn mgn_session_free(s: *mut mgn_session);
        pub fn mgn_session_last_error(s: *const mgn_session) -> *const c_char;
        pub fn mgn_session_num_dispatches(s: *const mgn_session) -> usize;
        pub fn mgn_session_dispatch_info(s: *const mgn_session, index: usize, out: *mut mgn_dispatch_info) -> mgn_status;
        pub fn mgn_session_set_parameter(s: *mut mgn_session, name: *const c_char, data: *const f32, len: usize) -> mgn_status;
        pub fn mgn_session_set_input(s: *mut mgn_session, name: *const c_char, data: *const f32, len: usize) -> mgn_status;
        pub fn mgn_session_step(s: *mut mgn_session) -> mgn_status;
        pub fn mgn_session_wait(s: *mut mgn_session) -> mgn_status;
        pub fn mgn_session_set_graph_replay(s: *mut mgn_session, enable: c_int) -> mgn_status;
        pub fn mgn_session_set_fusion(s: *mut mgn_session, enable: c_int) -> mgn_status;
        pub fn mgn_session_set_chains(s: *mut mgn_session, enable: c_int) -> mgn_status;
        pub fn mgn_session_num_launches(s: *mut mgn_session) -> usize;
        pub fn mgn_session_graph_active(s: *const mgn_session) -> c_int;
        pub fn mgn_session_read_output(s: *mut mgn_session, out: *mut f32, len: usize) -> mgn_status;
        pub fn mgn_session_read_output_by_index(s: *mut mgn_session, index: usize, out: *mut f32, len: usize) -> mgn_status;
        pub fn mgn_session_ctx(s: *mut mgn_session) -> *mut mgn_ctx;
    }
}
