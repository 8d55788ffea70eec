//! Raw bindings of the C ABI in `include/strix_mi355.h` (the counterpart of
//! crates/strix-backend-rocm/src/ffi.rs).  Return convention of every `c_int` function:
//! 1 done, 0 key / layer not resident, < 0 error (text in `smx_last_error`).

#![allow(dead_code)]

use std::os::raw::{c_char, c_float, c_int, c_void};

#[repr(C)]
pub struct SmxCtx {
    _private: [u8; 0],
}

extern "C" {
    pub fn smx_create(device: c_int, out: *mut *mut SmxCtx) -> c_int;
    pub fn smx_destroy(ctx: *mut SmxCtx);
    pub fn smx_last_error(ctx: *const SmxCtx) -> *const c_char;
    pub fn smx_name(ctx: *const SmxCtx) -> *const c_char;
    pub fn smx_resident_count(ctx: *const SmxCtx) -> usize;
    pub fn smx_resident_bytes(ctx: *const SmxCtx) -> usize;

    pub fn smx_upload_q4_0(
        ctx: *mut SmxCtx,
        key: *const c_char,
        bytes: *const c_void,
        nbytes: usize,
        in_dim: usize,
        out_dim: usize,
    ) -> c_int;
    pub fn smx_upload_q8_0(
        ctx: *mut SmxCtx,
        key: *const c_char,
        bytes: *const c_void,
        nbytes: usize,
        in_dim: usize,
        out_dim: usize,
    ) -> c_int;
    pub fn smx_upload_q6_k(
        ctx: *mut SmxCtx,
        key: *const c_char,
        bytes: *const c_void,
        nbytes: usize,
        in_dim: usize,
        out_dim: usize,
    ) -> c_int;
    pub fn smx_upload_moe_q8(
        ctx: *mut SmxCtx,
        layer: usize,
        gate: *const c_void,
        gate_nbytes: usize,
        up: *const c_void,
        up_nbytes: usize,
        down: *const c_void,
        down_nbytes: usize,
        hidden: usize,
        eff: usize,
        ne: usize,
    ) -> c_int;
    pub fn smx_upload_moe_q6(
        ctx: *mut SmxCtx,
        layer: usize,
        gate: *const c_void,
        gate_nbytes: usize,
        up: *const c_void,
        up_nbytes: usize,
        down: *const c_void,
        down_nbytes: usize,
        hidden: usize,
        eff: usize,
        ne: usize,
    ) -> c_int;
    pub fn smx_evict(ctx: *mut SmxCtx, key: *const c_char) -> c_int;
    pub fn smx_weight_dims(
        ctx: *const SmxCtx,
        key: *const c_char,
        in_dim: *mut usize,
        out_dim: *mut usize,
    ) -> c_int;

    pub fn smx_gemv(
        ctx: *mut SmxCtx,
        key: *const c_char,
        x: *const c_float,
        in_len: usize,
        y: *mut c_float,
        out_cap: usize,
    ) -> c_int;
    pub fn smx_gemv_f32(
        ctx: *mut SmxCtx,
        key: *const c_char,
        x: *const c_float,
        in_len: usize,
        y: *mut c_float,
        out_cap: usize,
    ) -> c_int;
    pub fn smx_gemv_rows(
        ctx: *mut SmxCtx,
        key: *const c_char,
        xs: *const c_float,
        m: usize,
        in_dim: usize,
        y: *mut c_float,
        y_cap: usize,
    ) -> c_int;
    pub fn smx_gemv_batch(
        ctx: *mut SmxCtx,
        n: usize,
        keys: *const *const c_char,
        xs: *const *const c_float,
        in_lens: *const usize,
        ys: *const *mut c_float,
        out_caps: *const usize,
        status: *mut c_int,
    ) -> c_int;
    pub fn smx_gemv_f32_batch(
        ctx: *mut SmxCtx,
        n: usize,
        keys: *const *const c_char,
        xs: *const *const c_float,
        in_lens: *const usize,
        ys: *const *mut c_float,
        out_caps: *const usize,
        status: *mut c_int,
    ) -> c_int;
    pub fn smx_gemm(
        ctx: *mut SmxCtx,
        key: *const c_char,
        xs: *const c_float,
        m: usize,
        in_dim: usize,
        y: *mut c_float,
        y_cap: usize,
    ) -> c_int;
    pub fn smx_lm_head_argmax_rows(
        ctx: *mut SmxCtx,
        key: *const c_char,
        xs: *const c_float,
        m: usize,
        in_dim: usize,
        out: *mut u32,
    ) -> c_int;

    pub fn smx_moe_ffn(
        ctx: *mut SmxCtx,
        layer: usize,
        ids: *const i32,
        wexp: *const c_float,
        k: usize,
        x: *const c_float,
        x_len: usize,
        sgate: c_float,
        y: *mut c_float,
        y_cap: usize,
    ) -> c_int;
    pub fn smx_moe_layer(
        ctx: *mut SmxCtx,
        layer: usize,
        xs: *const c_float,
        m: usize,
        plan: *const usize,
        nplan: usize,
        slot_tok: *const i32,
        wslot: *const c_float,
        slots: usize,
        y: *mut c_float,
        y_cap: usize,
    ) -> c_int;
    pub fn smx_moe_layer_ffn(
        ctx: *mut SmxCtx,
        layer: usize,
        plan: *const i32,
        nplan: usize,
        xs: *const c_float,
        rows: usize,
        dy: *mut c_float,
        dy_cap: usize,
    ) -> c_int;
    pub fn smx_moe_expert_ffn(
        ctx: *mut SmxCtx,
        layer: usize,
        expert: usize,
        xs: *const c_float,
        m: usize,
        y: *mut c_float,
        y_cap: usize,
    ) -> c_int;
    pub fn smx_moe_route(
        ctx: *mut SmxCtx,
        logits: *const c_float,
        ne: usize,
        k: usize,
        ids: *mut i32,
        w: *mut c_float,
    ) -> c_int;
}
