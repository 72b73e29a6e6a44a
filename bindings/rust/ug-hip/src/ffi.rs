//! `extern "C"` declarations of `include/ughip.h`, one for one: same names, same argument order.
//! `tests/test_rust_bindings.py` parses the header and this file and fails on any difference in
//! name, arity or argument type, so the two cannot drift apart unnoticed.
#![allow(non_camel_case_types)]
use std::ffi::{c_char, c_int, c_uint, c_void};

/// `ughip_a`: `ssa::A` on the wire (ug-core/src/lang.rs:642-646).
#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct UghipA {
    pub is_const: u8,
    pub dtype: u8,
    pub pad_: u16,
    pub var: u32,
    pub i: i64,
    pub f: f32,
    pub pad2_: u32,
}

/// `ughip_instr`: one `ssa::Instr` (ug-core/src/lang.rs:690-709); `op` is the discriminant in
/// declaration order, the other fields are used as the `UGHIP_I_*` comments of the header say.
#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct UghipInstr {
    pub op: i32,
    pub dtype: i32,
    pub sub: i32,
    pub v: u32,
    pub n: u64,
    pub a: UghipA,
    pub b: UghipA,
}

/// `ughip_kernel_arg`: one `(Arg, line_no)` of `ssa::Kernel::args()`.
#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct UghipKernelArg {
    pub arg_id: u64,
    pub is_ptr: u8,
    pub dtype: u8,
    pub pad_: u16,
    pub var: u32,
}

/// `ughip_ssa`: `ssa::Kernel` as a flat POD image.
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct UghipSsa {
    pub instrs: *const UghipInstr,
    pub n_instrs: usize,
    pub args: *const UghipKernelArg,
    pub n_args: usize,
    pub grid_dim: u32,
    pub block_dim: u32,
    pub shared_mem: u32,
    pub pad_: u32,
}

/// `ughip_func_info`: the lowering strategy and launch shape the backend picked.
#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct UghipFuncInfo {
    pub strategy: i32,
    pub grid_dim: u32,
    pub block_dim: u32,
    pub lds_bytes: u32,
    pub scratch_bytes: u64,
}

// Opaque handles.
pub enum UghipDevice {}
pub enum UghipSlice {}
pub enum UghipFunc {}
pub enum UghipEvent {}

// `UGHIP_*` dtype codes: the order of `ug::DType` (ug-core/src/dtype.rs:5-11).
pub const UGHIP_BF16: c_int = 0;
pub const UGHIP_F16: c_int = 1;
pub const UGHIP_F32: c_int = 2;
pub const UGHIP_I32: c_int = 3;
pub const UGHIP_I64: c_int = 4;

/// Size of the static device array behind `ughip_matmul_noalloc`.
pub const UGHIP_PRODUCT_F32: c_int = 0;
pub const UGHIP_PRODUCT_BF16X3: c_int = 1;
pub const UGHIP_MATMUL_NOALLOC_SCRATCH_BYTES: usize = 64 << 20;

extern "C" {
    pub fn ughip_last_error() -> *const c_char;
    pub fn ughip_last_kernel() -> *const c_char;
    pub fn ughip_device_create(ordinal: c_int, out: *mut *mut UghipDevice) -> c_int;
    pub fn ughip_device_retain(dev: *mut UghipDevice) -> c_int;
    pub fn ughip_device_release(dev: *mut UghipDevice) -> c_int;
    pub fn ughip_synchronize(dev: *mut UghipDevice) -> c_int;
    pub fn ughip_device_arch(dev: *mut UghipDevice, buf: *mut c_char, buf_len: usize) -> c_int;
    pub fn ughip_device_stats(
        dev: *mut UghipDevice,
        n_code_objects: *mut usize,
        pool_bytes: *mut usize,
        live_bytes: *mut usize,
    ) -> c_int;
    pub fn ughip_use_grid() -> c_int;
    pub fn ughip_alloc(dev: *mut UghipDevice, dtype: c_int, len: usize, out: *mut *mut UghipSlice) -> c_int;
    pub fn ughip_device_set_zero_fill(dev: *mut UghipDevice, on: c_int) -> c_int;
    pub fn ughip_free(s: *mut UghipSlice) -> c_int;
    pub fn ughip_slice_len(s: *const UghipSlice) -> usize;
    pub fn ughip_slice_dtype(s: *const UghipSlice) -> c_int;
    pub fn ughip_slice_ptr(s: *const UghipSlice) -> *mut c_void;
    pub fn ughip_h2d(dst: *mut UghipSlice, src: *const c_void, dtype: c_int, len: usize) -> c_int;
    pub fn ughip_d2h(src: *const UghipSlice, dst: *mut c_void, dtype: c_int, len: usize) -> c_int;
    pub fn ughip_compile(
        dev: *mut UghipDevice,
        ssa: *const UghipSsa,
        name: *const c_char,
        out: *mut *mut UghipFunc,
    ) -> c_int;
    pub fn ughip_func_release(f: *mut UghipFunc) -> c_int;
    pub fn ughip_run(dev: *mut UghipDevice, f: *mut UghipFunc, args: *const *mut UghipSlice, n_args: usize) -> c_int;
    pub fn ughip_run_part(
        dev: *mut UghipDevice,
        f: *mut UghipFunc,
        args: *const *mut UghipSlice,
        n_args: usize,
        part: c_int,
    ) -> c_int;
    pub fn ughip_func_source(f: *const UghipFunc, buf: *mut c_char, buf_len: usize) -> usize;
    pub fn ughip_func_get_info(f: *const UghipFunc, out: *mut UghipFuncInfo) -> c_int;
    pub fn ughip_codegen(
        ssa: *const UghipSsa,
        name: *const c_char,
        buf: *mut c_char,
        buf_len: usize,
        out_len: *mut usize,
        info: *mut UghipFuncInfo,
    ) -> c_int;
    pub fn ughip_matmul_plan(
        dtype: c_int,
        rhs_dtype: c_int,
        b: usize,
        m: usize,
        n: usize,
        k: usize,
        rhs_nk: c_int,
        buf: *mut c_char,
        buf_len: usize,
    ) -> c_int;
    pub fn ughip_set_tuning(name: *const c_char, set: c_int, value: i64) -> c_int;
    pub fn ughip_codegen_min_len(ssa: *const UghipSsa, min_len: *mut i64, n_args: usize) -> c_int;
    pub fn ughip_codegen_as_written(
        ssa: *const UghipSsa,
        name: *const c_char,
        buf: *mut c_char,
        buf_len: usize,
        out_len: *mut usize,
    ) -> c_int;
    pub fn ughip_compile_source(
        dev: *mut UghipDevice,
        source: *const c_char,
        entry: *const c_char,
        n_args: usize,
        arg_dtypes: *const c_int,
        grid_dim: c_uint,
        block_dim: c_uint,
        shared_mem_bytes: c_uint,
        out: *mut *mut UghipFunc,
    ) -> c_int;
    pub fn ughip_rtc_check(source: *const c_char, arch: *const c_char, code_size: *mut usize) -> c_int;
    pub fn ughip_matmul(
        dev: *mut UghipDevice,
        dst: *mut UghipSlice,
        lhs: *const UghipSlice,
        rhs: *const UghipSlice,
        b: usize,
        m: usize,
        n: usize,
        k: usize,
        rank: usize,
        lhs_dims: *const usize,
        lhs_strides: *const usize,
        lhs_offset: usize,
        rhs_dims: *const usize,
        rhs_strides: *const usize,
        rhs_offset: usize,
    ) -> c_int;
    pub fn ughip_matmul_noalloc(
        dev: *mut UghipDevice,
        dst: *mut UghipSlice,
        lhs: *const UghipSlice,
        rhs: *const UghipSlice,
        b: usize,
        m: usize,
        n: usize,
        k: usize,
        rank: usize,
        lhs_dims: *const usize,
        lhs_strides: *const usize,
        lhs_offset: usize,
        rhs_dims: *const usize,
        rhs_strides: *const usize,
        rhs_offset: usize,
    ) -> c_int;
    pub fn ughip_rope(
        dev: *mut UghipDevice,
        src: *const UghipSlice,
        cos: *const UghipSlice,
        sin: *const UghipSlice,
        pos: *const UghipSlice,
        dst: *mut UghipSlice,
        bh: usize,
        t: usize,
        d: usize,
        interleaved: c_int,
    ) -> c_int;
    pub fn ughip_cat(
        dev: *mut UghipDevice,
        lhs: *const UghipSlice,
        rhs: *const UghipSlice,
        dst: *mut UghipSlice,
        d1: usize,
        d2_l: usize,
        d2_r: usize,
    ) -> c_int;
    pub fn ughip_softmax_rows(
        dev: *mut UghipDevice,
        src: *const UghipSlice,
        dst: *mut UghipSlice,
        n_rows: usize,
        n_cols: usize,
    ) -> c_int;
    pub fn ughip_causal_mask(
        dev: *mut UghipDevice,
        src: *const UghipSlice,
        dst: *mut UghipSlice,
        bh: usize,
        s1: usize,
        s2: usize,
    ) -> c_int;
    pub fn ughip_causal_softmax_rows(
        dev: *mut UghipDevice,
        src: *const UghipSlice,
        dst: *mut UghipSlice,
        bh: usize,
        s1: usize,
        s2: usize,
    ) -> c_int;
    pub fn ughip_attention_decode(
        dev: *mut UghipDevice,
        q: *const UghipSlice,
        k: *const UghipSlice,
        v: *const UghipSlice,
        dst: *mut UghipSlice,
        b: usize,
        n_heads: usize,
        n_kv_heads: usize,
        s: usize,
        d: usize,
        scale: f32,
    ) -> c_int;
    pub fn ughip_attention_decode_rope(
        dev: *mut UghipDevice,
        q: *const UghipSlice,
        k: *const UghipSlice,
        v: *const UghipSlice,
        dst: *mut UghipSlice,
        b: usize,
        n_heads: usize,
        n_kv_heads: usize,
        s: usize,
        d: usize,
        scale: f32,
        cos: *const UghipSlice,
        sin: *const UghipSlice,
        pos: *const UghipSlice,
        interleaved: c_int,
    ) -> c_int;
    pub fn ughip_rope_append(
        dev: *mut UghipDevice,
        cache: *const UghipSlice,
        x: *const UghipSlice,
        dst: *mut UghipSlice,
        bh: usize,
        s_old: usize,
        d: usize,
        cos: *const UghipSlice,
        sin: *const UghipSlice,
        pos: *const UghipSlice,
        interleaved: c_int,
    ) -> c_int;
    pub fn ughip_kv_append(
        dev: *mut UghipDevice,
        cache: *mut UghipSlice,
        x: *const UghipSlice,
        x_offset: usize,
        x_row_stride: usize,
        b: usize,
        n: usize,
        cap: usize,
        s_old: usize,
        t: usize,
        d: usize,
        cos: *const UghipSlice,
        sin: *const UghipSlice,
        pos: *const UghipSlice,
        interleaved: c_int,
    ) -> c_int;
    pub fn ughip_kv_append_pair(
        dev: *mut UghipDevice,
        kcache: *mut UghipSlice,
        vcache: *mut UghipSlice,
        x: *const UghipSlice,
        k_offset: usize,
        v_offset: usize,
        x_row_stride: usize,
        b: usize,
        n: usize,
        cap: usize,
        s_old: usize,
        t: usize,
        d: usize,
        cos: *const UghipSlice,
        sin: *const UghipSlice,
        pos: *const UghipSlice,
        interleaved: c_int,
    ) -> c_int;
    pub fn ughip_attention_cached(
        dev: *mut UghipDevice,
        q: *const UghipSlice,
        q_offset: usize,
        q_row_stride: usize,
        k: *const UghipSlice,
        v: *const UghipSlice,
        dst: *mut UghipSlice,
        b: usize,
        n_heads: usize,
        n_kv_heads: usize,
        t: usize,
        s: usize,
        cap: usize,
        d: usize,
        scale: f32,
        cos: *const UghipSlice,
        sin: *const UghipSlice,
        pos: *const UghipSlice,
        interleaved: c_int,
    ) -> c_int;
    pub fn ughip_attention_cached_linear_add_rows(
        dev: *mut UghipDevice,
        q: *const UghipSlice,
        q_offset: usize,
        q_row_stride: usize,
        k: *const UghipSlice,
        v: *const UghipSlice,
        b: usize,
        n_heads: usize,
        n_kv_heads: usize,
        t: usize,
        s: usize,
        cap: usize,
        d: usize,
        scale: f32,
        cos: *const UghipSlice,
        sin: *const UghipSlice,
        pos: *const UghipSlice,
        interleaved: c_int,
        w: *const UghipSlice,
        residual: *const UghipSlice,
        dst: *mut UghipSlice,
        n: usize,
        product: c_int,
    ) -> c_int;
    pub fn ughip_attention_step(
        dev: *mut UghipDevice,
        qkv: *const UghipSlice,
        row_stride: usize,
        q_offset: usize,
        k_offset: usize,
        v_offset: usize,
        kcache: *mut UghipSlice,
        vcache: *mut UghipSlice,
        dst: *mut UghipSlice,
        b: usize,
        n_heads: usize,
        n_kv_heads: usize,
        s_old: usize,
        cap: usize,
        d: usize,
        scale: f32,
        cos: *const UghipSlice,
        sin: *const UghipSlice,
        pos: *const UghipSlice,
        interleaved: c_int,
    ) -> c_int;
    pub fn ughip_gemv_multi(
        dev: *mut UghipDevice,
        x: *const UghipSlice,
        n_mats: usize,
        w: *const *const UghipSlice,
        n: *const usize,
        k: usize,
        dst: *mut UghipSlice,
    ) -> c_int;
    pub fn ughip_gemv_gate_up(
        dev: *mut UghipDevice,
        x: *const UghipSlice,
        w_gate: *const UghipSlice,
        w_up: *const UghipSlice,
        dst: *mut UghipSlice,
        n: usize,
        k: usize,
    ) -> c_int;
    pub fn ughip_rms_gemv_multi(
        dev: *mut UghipDevice,
        x: *const UghipSlice,
        alpha: *const UghipSlice,
        eps: f32,
        n_mats: usize,
        w: *const *const UghipSlice,
        n: *const usize,
        k: usize,
        dst: *mut UghipSlice,
    ) -> c_int;
    pub fn ughip_rms_gemv_gate_up(
        dev: *mut UghipDevice,
        x: *const UghipSlice,
        alpha: *const UghipSlice,
        eps: f32,
        w_gate: *const UghipSlice,
        w_up: *const UghipSlice,
        dst: *mut UghipSlice,
        n: usize,
        k: usize,
    ) -> c_int;
    pub fn ughip_gemv_add(
        dev: *mut UghipDevice,
        x: *const UghipSlice,
        w: *const UghipSlice,
        residual: *const UghipSlice,
        dst: *mut UghipSlice,
        n: usize,
        k: usize,
    ) -> c_int;
    pub fn ughip_linear_rows(
        dev: *mut UghipDevice,
        x: *const UghipSlice,
        w: *const UghipSlice,
        dst: *mut UghipSlice,
        m: usize,
        n: usize,
        k: usize,
        product: c_int,
    ) -> c_int;
    pub fn ughip_linear_add_rows(
        dev: *mut UghipDevice,
        x: *const UghipSlice,
        w: *const UghipSlice,
        residual: *const UghipSlice,
        dst: *mut UghipSlice,
        m: usize,
        n: usize,
        k: usize,
        product: c_int,
    ) -> c_int;
    pub fn ughip_linear_swiglu_rows(
        dev: *mut UghipDevice,
        x: *const UghipSlice,
        w: *const UghipSlice,
        dst: *mut UghipSlice,
        m: usize,
        n: usize,
        k: usize,
        product: c_int,
    ) -> c_int;
    pub fn ughip_rms_linear_rows(
        dev: *mut UghipDevice,
        x: *const UghipSlice,
        alpha: *const UghipSlice,
        eps: f32,
        w: *const UghipSlice,
        dst: *mut UghipSlice,
        m: usize,
        n: usize,
        k: usize,
        product: c_int,
    ) -> c_int;
    pub fn ughip_rms_mlp_rows(
        dev: *mut UghipDevice,
        x: *const UghipSlice,
        alpha: *const UghipSlice,
        eps: f32,
        w_gate_up: *const UghipSlice,
        w_down: *const UghipSlice,
        residual: *const UghipSlice,
        dst: *mut UghipSlice,
        m: usize,
        n: usize,
        inter: usize,
        k: usize,
        product: c_int,
    ) -> c_int;
    pub fn ughip_linear_rows_plan(
        w_dtype: c_int,
        product: c_int,
        form: c_int,
        m: usize,
        n: usize,
        k: usize,
        buf: *mut c_char,
        buf_len: usize,
    ) -> c_int;
    pub fn ughip_argmax_row(
        dev: *mut UghipDevice,
        logits: *const UghipSlice,
        n: usize,
        row: usize,
        token: *mut UghipSlice,
        ids: *mut UghipSlice,
        vals: *mut UghipSlice,
        slot: usize,
    ) -> c_int;
    pub fn ughip_convert(dev: *mut UghipDevice, src: *const UghipSlice, dst: *mut UghipSlice) -> c_int;
    pub fn ughip_event_create(dev: *mut UghipDevice, out: *mut *mut UghipEvent) -> c_int;
    pub fn ughip_event_record(ev: *mut UghipEvent) -> c_int;
    pub fn ughip_event_elapsed_ms(start: *mut UghipEvent, stop: *mut UghipEvent, ms: *mut f32) -> c_int;
    pub fn ughip_event_destroy(ev: *mut UghipEvent) -> c_int;
}

/// Maps a return code to `ug::Result`, with the library's thread-local message.
pub fn check(rc: c_int) -> ug::Result<()> {
    if rc == 0 {
        return Ok(());
    }
    let msg = unsafe { std::ffi::CStr::from_ptr(ughip_last_error()) }.to_string_lossy().into_owned();
    Err(ug::Error::Msg(format!("ughip error {rc}: {msg}")).bt())
}
