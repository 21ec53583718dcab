//! Raw FFI of the MI355X (gfx950) mixture-of-experts layer library, `include/atenia_moe_hip.h`.
//!
//! Takes the place of `src/cuda` for the MoE layer path.  Same discipline as the reference's CUDA
//! bindings (`src/cuda/matmul.rs:21-51`, `src/cuda/int8_to_bf16.rs:63-145`): the real symbols are
//! declared under `#[cfg(atenia_hip)]`, which `build.rs` sets only after hipcc has compiled and
//! archived every kernel; without it every symbol has an identical-signature stub, so a host
//! without ROCm still links.  The stubs are unreachable by construction: `available()` answers
//! `false` there and the safe wrappers below return `Err` before any of them is called.
//!
//! Every function returns the library's `int` code: 0 ok; 1 sync failed; 2 launch failed; -1 bad
//! dimensions; -2 bad k; -3 non-finite routing weight; -4 out of device memory; -5 bad handle;
//! -6 unsupported.  No unwinding crosses the boundary.
#![allow(non_camel_case_types)]

use std::ffi::CStr;
use std::os::raw::{c_char, c_int, c_void};

pub const ATENIA_MOE_CONVENTION_ATENIA: i32 = 0;
pub const ATENIA_MOE_CONVENTION_HUGGINGFACE_QWEN: i32 = 1;
pub const ATENIA_MOE_WEIGHT_F32: i32 = 0;
pub const ATENIA_MOE_WEIGHT_BF16: i32 = 1;
pub const ATENIA_MOE_WEIGHT_INT8_W8A16: i32 = 2;
pub const ATENIA_MOE_WEIGHT_INT8_PER_GROUP: i32 = 3;
pub const ATENIA_MOE_ACT_F32: c_int = 0;
pub const ATENIA_MOE_ACT_BF16: c_int = 1;
pub const ATENIA_MOE_NORM_GRAPH_F32: c_int = 0;
pub const ATENIA_MOE_NORM_F64: c_int = 1;
pub const ATENIA_MOE_POLICY_CERTIFIED: c_int = 0;
pub const ATENIA_MOE_POLICY_STRICT: c_int = 1;
pub const ATENIA_MOE_POLICY_FAST: c_int = 2;
pub const ATENIA_MOE_N_STAGES: usize = 6;
pub const ATENIA_MOE_KERNELS_STREAM: i32 = 0;
pub const ATENIA_MOE_KERNELS_MID: i32 = 1;
pub const ATENIA_MOE_KERNELS_TILED: i32 = 2;
pub const ATENIA_MOE_KERNELS_F32: i32 = 3;

pub const ATENIA_MOE_OK: c_int = 0;
pub const ATENIA_MOE_ERR_SYNC: c_int = 1;
pub const ATENIA_MOE_ERR_LAUNCH: c_int = 2;
pub const ATENIA_MOE_ERR_DIM: c_int = -1;
pub const ATENIA_MOE_ERR_K: c_int = -2;
pub const ATENIA_MOE_ERR_NON_FINITE: c_int = -3;
pub const ATENIA_MOE_ERR_OOM: c_int = -4;
pub const ATENIA_MOE_ERR_HANDLE: c_int = -5;
pub const ATENIA_MOE_ERR_UNSUPPORTED: c_int = -6;

/// Opaque handle; owns the layer's weights and workspace in HBM.
#[repr(C)]
pub struct AteniaMoeLayer {
    _private: [u8; 0],
}

/// Field for field the C struct of the same name.  All pointers are host pointers borrowed for
/// the duration of `atenia_moe_hip_layer_create`.
#[repr(C)]
pub struct AteniaMoeLayerDesc {
    pub num_experts: i32,
    pub top_k: i32,
    pub d_model: i32,
    pub d_ff: i32,
    pub d_ff_shared: i32,
    pub convention: i32,
    pub weight_dtype: i32,
    pub max_tokens_hint: i32,
    pub w_router: *const f32,
    pub router_bias: *const f32,
    pub w_gate: *const c_void,
    pub w_up: *const c_void,
    pub w_down: *const c_void,
    pub scale_gate: *const f32,
    pub scale_up: *const f32,
    pub scale_down: *const f32,
    pub s_gate: *const c_void,
    pub s_up: *const c_void,
    pub s_down: *const c_void,
    pub s_scale_gate: *const f32,
    pub s_scale_up: *const f32,
    pub s_scale_down: *const f32,
    pub shared_gate: *const f32,
    pub group_size: i32,
}

#[cfg(atenia_hip)]
#[link(name = "atenia_moe_hip", kind = "static")]
unsafe extern "C" {
    pub fn atenia_moe_hip_available() -> c_int;
    pub fn atenia_moe_hip_last_error_string() -> *const c_char;
    pub fn atenia_moe_quantize_per_group_i8(
        w: *const f32,
        rows: usize,
        cols: usize,
        group_size: usize,
        q_out: *mut i8,
        scales_out: *mut f32,
    ) -> c_int;
    pub fn atenia_moe_hip_layer_create(
        desc: *const AteniaMoeLayerDesc,
        out_layer: *mut *mut AteniaMoeLayer,
    ) -> c_int;
    pub fn atenia_moe_hip_layer_destroy(layer: *mut AteniaMoeLayer) -> c_int;
    pub fn atenia_moe_hip_layer_forward(
        layer: *mut AteniaMoeLayer,
        x_host: *const f32,
        n_tokens: c_int,
        out_host: *mut f32,
    ) -> c_int;
    pub fn atenia_moe_hip_layer_forward_device(
        layer: *mut AteniaMoeLayer,
        d_x: *const c_void,
        x_dtype: c_int,
        n_tokens: c_int,
        d_out: *mut f32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn atenia_moe_hip_layer_forward_device_noalloc(
        layer: *mut AteniaMoeLayer,
        d_x: *const c_void,
        x_dtype: c_int,
        n_tokens: c_int,
        d_out: *mut f32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn atenia_moe_hip_layer_set_v3_router(
        layer: *mut AteniaMoeLayer,
        n_group: c_int,
        topk_group: c_int,
        routed_scaling_factor: f64,
        norm_topk_prob: c_int,
        e_score_correction_bias_host: *const f32,
    ) -> c_int;
    pub fn atenia_moe_hip_layer_block_forward_device(
        layer: *mut AteniaMoeLayer,
        d_x1: *const f32,
        n_tokens: c_int,
        d_gamma: *const f32,
        eps: f32,
        norm_policy: c_int,
        d_out: *mut f32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn atenia_moe_hip_layer_block_forward(
        layer: *mut AteniaMoeLayer,
        x1_host: *const f32,
        n_tokens: c_int,
        gamma_host: *const f32,
        eps: f32,
        norm_policy: c_int,
        out_host: *mut f32,
    ) -> c_int;
    pub fn atenia_moe_hip_layer_status(
        layer: *mut AteniaMoeLayer,
        stream: *mut c_void,
        token: *mut i32,
        expert: *mut i32,
    ) -> c_int;
    pub fn atenia_moe_hip_layer_last_non_finite(
        layer: *mut AteniaMoeLayer,
        token: *mut i32,
        expert: *mut i32,
    ) -> c_int;
    pub fn atenia_moe_hip_layer_route(
        layer: *mut AteniaMoeLayer,
        x_host: *const f32,
        n_tokens: c_int,
        idx_host: *mut i32,
        w_host: *mut f32,
    ) -> c_int;
    pub fn atenia_moe_hip_layer_permute(
        layer: *mut AteniaMoeLayer,
        idx_host: *const i32,
        n_tokens: c_int,
        counts_host: *mut i32,
        offsets_host: *mut i32,
        perm_host: *mut i32,
    ) -> c_int;
    pub fn atenia_moe_router_launch_device(
        layer: *mut AteniaMoeLayer,
        d_x: *const c_void,
        x_dtype: c_int,
        n_tokens: c_int,
        d_idx: *mut i32,
        d_w: *mut f32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn atenia_moe_permute_launch_device(
        layer: *mut AteniaMoeLayer,
        n_tokens: c_int,
        d_counts: *mut i32,
        d_offsets: *mut i32,
        d_perm: *mut i32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn atenia_moe_expert_ffn_launch_device(
        layer: *mut AteniaMoeLayer,
        d_x: *const c_void,
        x_dtype: c_int,
        n_tokens: c_int,
        stream: *mut c_void,
    ) -> c_int;
    pub fn atenia_moe_combine_launch_device(
        layer: *mut AteniaMoeLayer,
        n_tokens: c_int,
        d_out: *mut f32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn atenia_moe_hip_layer_last_routing(
        layer: *mut AteniaMoeLayer,
        idx_host: *mut i32,
        w_host: *mut f32,
        counts_host: *mut i32,
        offsets_host: *mut i32,
        perm_host: *mut i32,
    ) -> c_int;
    pub fn atenia_moe_hip_layer_last_expert_outputs(
        layer: *mut AteniaMoeLayer,
        y_host: *mut f32,
        y_shared_host: *mut f32,
    ) -> c_int;
    pub fn atenia_moe_hip_layer_last_down_split(
        layer: *mut AteniaMoeLayer,
        parts_host: *mut u8,
    ) -> c_int;
    pub fn atenia_moe_hip_layer_last_normed(layer: *mut AteniaMoeLayer, h2_host: *mut f32) -> c_int;
    pub fn atenia_moe_hip_layer_set_profiling(layer: *mut AteniaMoeLayer, enabled: c_int) -> c_int;
    pub fn atenia_moe_hip_layer_stage_ms(layer: *mut AteniaMoeLayer, ms: *mut f32) -> c_int;
    pub fn atenia_moe_hip_layer_stage_launches(layer: *mut AteniaMoeLayer, n: *mut i32) -> c_int;
    pub fn atenia_moe_hip_layer_set_numeric_policy(
        layer: *mut AteniaMoeLayer,
        policy: c_int,
    ) -> c_int;
    pub fn atenia_moe_hip_layer_info(layer: *const AteniaMoeLayer, info: *mut i64) -> c_int;
    pub fn atenia_moe_hip_layer_expert_kernels(
        layer: *const AteniaMoeLayer,
        n_tokens: i64,
        family: *mut i32,
    ) -> c_int;
    pub fn atenia_moe_hip_plan_batch(
        num_experts: c_int,
        top_k: c_int,
        d_model: c_int,
        d_ff: c_int,
        d_ff_shared: c_int,
        weight_dtype: c_int,
        group_size: c_int,
        n_tokens: i64,
        plan: *mut i32,
    ) -> c_int;
    pub fn atenia_moe_quantize_per_row_i8(
        w: *const f32,
        rows: usize,
        cols: usize,
        q: *mut i8,
        scales: *mut f32,
    ) -> c_int;
    pub fn atenia_moe_absmax_per_channel_symmetric(
        w: *const f32,
        k: usize,
        n: usize,
        q: *mut i8,
        scales: *mut f32,
    ) -> c_int;
    pub fn atenia_moe_absmax_per_group_symmetric(
        w: *const f32,
        k: usize,
        n: usize,
        group_size: usize,
        q: *mut i8,
        scales: *mut f32,
    ) -> c_int;
    pub fn atenia_moe_f32_to_bf16_trunc(src: *const f32, n: usize, dst: *mut u16) -> c_int;
    pub fn atenia_moe_int8_to_bf16_per_channel_launch_device(
        d_int8: *const c_void,
        d_scales: *const f32,
        d_bf16: *mut c_void,
        k: c_int,
        n: c_int,
        stream: *mut c_void,
    ) -> c_int;
    pub fn atenia_moe_int8_to_bf16_per_group_launch_device(
        d_int8: *const c_void,
        d_scales: *const f32,
        d_bf16: *mut c_void,
        k: c_int,
        n: c_int,
        group_size: c_int,
        stream: *mut c_void,
    ) -> c_int;
    pub fn int8_to_bf16_per_channel_launch_device(
        d_int8: *const c_void,
        d_scales: *const f32,
        d_bf16: *mut c_void,
        k: c_int,
        n: c_int,
    ) -> c_int;
    pub fn int8_to_bf16_per_group_launch_device(
        d_int8: *const c_void,
        d_scales: *const f32,
        d_bf16: *mut c_void,
        k: c_int,
        n: c_int,
        group_size: c_int,
    ) -> c_int;
}

// Builds without hipcc: no static library to link.  Identical-signature stubs.
#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_available() -> c_int {
    0
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_last_error_string() -> *const c_char {
    unreachable!("HIP symbol atenia_moe_hip_last_error_string called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_quantize_per_group_i8(
    w: *const f32,
    rows: usize,
    cols: usize,
    group_size: usize,
    q_out: *mut i8,
    scales_out: *mut f32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_quantize_per_group_i8 called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_create(
    desc: *const AteniaMoeLayerDesc,
    out_layer: *mut *mut AteniaMoeLayer,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_create called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_destroy(layer: *mut AteniaMoeLayer) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_destroy called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_forward(
    layer: *mut AteniaMoeLayer,
    x_host: *const f32,
    n_tokens: c_int,
    out_host: *mut f32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_forward called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_forward_device(
    layer: *mut AteniaMoeLayer,
    d_x: *const c_void,
    x_dtype: c_int,
    n_tokens: c_int,
    d_out: *mut f32,
    stream: *mut c_void,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_forward_device called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_forward_device_noalloc(
    layer: *mut AteniaMoeLayer,
    d_x: *const c_void,
    x_dtype: c_int,
    n_tokens: c_int,
    d_out: *mut f32,
    stream: *mut c_void,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_forward_device_noalloc called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_set_v3_router(
    layer: *mut AteniaMoeLayer,
    n_group: c_int,
    topk_group: c_int,
    routed_scaling_factor: f64,
    norm_topk_prob: c_int,
    e_score_correction_bias_host: *const f32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_set_v3_router called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_block_forward_device(
    layer: *mut AteniaMoeLayer,
    d_x1: *const f32,
    n_tokens: c_int,
    d_gamma: *const f32,
    eps: f32,
    norm_policy: c_int,
    d_out: *mut f32,
    stream: *mut c_void,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_block_forward_device called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_block_forward(
    layer: *mut AteniaMoeLayer,
    x1_host: *const f32,
    n_tokens: c_int,
    gamma_host: *const f32,
    eps: f32,
    norm_policy: c_int,
    out_host: *mut f32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_block_forward called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_status(
    layer: *mut AteniaMoeLayer,
    stream: *mut c_void,
    token: *mut i32,
    expert: *mut i32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_status called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_last_non_finite(
    layer: *mut AteniaMoeLayer,
    token: *mut i32,
    expert: *mut i32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_last_non_finite called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_route(
    layer: *mut AteniaMoeLayer,
    x_host: *const f32,
    n_tokens: c_int,
    idx_host: *mut i32,
    w_host: *mut f32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_route called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_permute(
    layer: *mut AteniaMoeLayer,
    idx_host: *const i32,
    n_tokens: c_int,
    counts_host: *mut i32,
    offsets_host: *mut i32,
    perm_host: *mut i32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_permute called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_router_launch_device(
    layer: *mut AteniaMoeLayer,
    d_x: *const c_void,
    x_dtype: c_int,
    n_tokens: c_int,
    d_idx: *mut i32,
    d_w: *mut f32,
    stream: *mut c_void,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_router_launch_device called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_permute_launch_device(
    layer: *mut AteniaMoeLayer,
    n_tokens: c_int,
    d_counts: *mut i32,
    d_offsets: *mut i32,
    d_perm: *mut i32,
    stream: *mut c_void,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_permute_launch_device called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_expert_ffn_launch_device(
    layer: *mut AteniaMoeLayer,
    d_x: *const c_void,
    x_dtype: c_int,
    n_tokens: c_int,
    stream: *mut c_void,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_expert_ffn_launch_device called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_combine_launch_device(
    layer: *mut AteniaMoeLayer,
    n_tokens: c_int,
    d_out: *mut f32,
    stream: *mut c_void,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_combine_launch_device called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_last_routing(
    layer: *mut AteniaMoeLayer,
    idx_host: *mut i32,
    w_host: *mut f32,
    counts_host: *mut i32,
    offsets_host: *mut i32,
    perm_host: *mut i32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_last_routing called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_last_expert_outputs(
    layer: *mut AteniaMoeLayer,
    y_host: *mut f32,
    y_shared_host: *mut f32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_last_expert_outputs called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_last_down_split(
    layer: *mut AteniaMoeLayer,
    parts_host: *mut u8,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_last_down_split called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_last_normed(
    layer: *mut AteniaMoeLayer,
    h2_host: *mut f32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_last_normed called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_set_profiling(
    layer: *mut AteniaMoeLayer,
    enabled: c_int,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_set_profiling called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_stage_ms(layer: *mut AteniaMoeLayer, ms: *mut f32) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_stage_ms called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_stage_launches(
    layer: *mut AteniaMoeLayer,
    n: *mut i32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_stage_launches called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_set_numeric_policy(
    layer: *mut AteniaMoeLayer,
    policy: c_int,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_set_numeric_policy called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_info(layer: *const AteniaMoeLayer, info: *mut i64) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_info called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_hip_layer_expert_kernels(
    layer: *const AteniaMoeLayer,
    n_tokens: i64,
    family: *mut i32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_layer_expert_kernels called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc, clippy::too_many_arguments)]
pub unsafe fn atenia_moe_hip_plan_batch(
    num_experts: c_int,
    top_k: c_int,
    d_model: c_int,
    d_ff: c_int,
    d_ff_shared: c_int,
    weight_dtype: c_int,
    group_size: c_int,
    n_tokens: i64,
    plan: *mut i32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_hip_plan_batch called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_quantize_per_row_i8(
    w: *const f32,
    rows: usize,
    cols: usize,
    q: *mut i8,
    scales: *mut f32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_quantize_per_row_i8 called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_absmax_per_channel_symmetric(
    w: *const f32,
    k: usize,
    n: usize,
    q: *mut i8,
    scales: *mut f32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_absmax_per_channel_symmetric called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_absmax_per_group_symmetric(
    w: *const f32,
    k: usize,
    n: usize,
    group_size: usize,
    q: *mut i8,
    scales: *mut f32,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_absmax_per_group_symmetric called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_f32_to_bf16_trunc(src: *const f32, n: usize, dst: *mut u16) -> c_int {
    unreachable!("HIP symbol atenia_moe_f32_to_bf16_trunc called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_int8_to_bf16_per_channel_launch_device(
    d_int8: *const c_void,
    d_scales: *const f32,
    d_bf16: *mut c_void,
    k: c_int,
    n: c_int,
    stream: *mut c_void,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_int8_to_bf16_per_channel_launch_device called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn atenia_moe_int8_to_bf16_per_group_launch_device(
    d_int8: *const c_void,
    d_scales: *const f32,
    d_bf16: *mut c_void,
    k: c_int,
    n: c_int,
    group_size: c_int,
    stream: *mut c_void,
) -> c_int {
    unreachable!("HIP symbol atenia_moe_int8_to_bf16_per_group_launch_device called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn int8_to_bf16_per_channel_launch_device(
    d_int8: *const c_void,
    d_scales: *const f32,
    d_bf16: *mut c_void,
    k: c_int,
    n: c_int,
) -> c_int {
    unreachable!("HIP symbol int8_to_bf16_per_channel_launch_device called in a build without atenia_hip")
}

#[cfg(not(atenia_hip))]
#[allow(unused_variables, clippy::missing_safety_doc)]
pub unsafe fn int8_to_bf16_per_group_launch_device(
    d_int8: *const c_void,
    d_scales: *const f32,
    d_bf16: *mut c_void,
    k: c_int,
    n: c_int,
    group_size: c_int,
) -> c_int {
    unreachable!("HIP symbol int8_to_bf16_per_group_launch_device called in a build without atenia_hip")
}

// ---- safe layer over the raw symbols ---------------------------------------------------------

/// `true` when the library was built (cfg `atenia_hip`) and a gfx950 device is usable.  The
/// probe runs once per process, like `cuda_available()` (`src/cuda/mod.rs:61-70`).
pub fn available() -> bool {
    use std::sync::OnceLock;
    static PROBE: OnceLock<bool> = OnceLock::new();
    *PROBE.get_or_init(|| cfg!(atenia_hip) && unsafe { atenia_moe_hip_available() } == 1)
}

/// A non-zero library code with the calling thread's error text.
#[derive(Debug, Clone, PartialEq, Eq)]
pub struct MoeHipError {
    pub code: c_int,
    pub message: String,
}

impl std::fmt::Display for MoeHipError {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        write!(f, "atenia_moe_hip rc={}: {}", self.code, self.message)
    }
}

impl std::error::Error for MoeHipError {}

fn check(code: c_int) -> Result<(), MoeHipError> {
    if code == ATENIA_MOE_OK {
        return Ok(());
    }
    let message = unsafe {
        let p = atenia_moe_hip_last_error_string();
        if p.is_null() { String::new() } else { CStr::from_ptr(p).to_string_lossy().into_owned() }
    };
    Err(MoeHipError { code, message })
}

fn unavailable() -> MoeHipError {
    MoeHipError { code: ATENIA_MOE_ERR_LAUNCH, message: "no gfx950 device or library built without hipcc".into() }
}

/// Owns one `AteniaMoeLayer*`; dropped = destroyed.  One handle is not re-entrant (the library
/// serialises calls on it); it may be moved to and used from any thread.
pub struct HipMoeLayer {
    raw: *mut AteniaMoeLayer,
    d_model: usize,
}

unsafe impl Send for HipMoeLayer {}
unsafe impl Sync for HipMoeLayer {}

impl HipMoeLayer {
    /// Uploads the layer described by `desc` (host pointers valid for this call).
    ///
    /// # Safety
    /// Every non-null pointer of `desc` must address as many elements as the header documents.
    pub unsafe fn create(desc: &AteniaMoeLayerDesc) -> Result<Self, MoeHipError> {
        if !available() {
            return Err(unavailable());
        }
        let mut raw: *mut AteniaMoeLayer = std::ptr::null_mut();
        check(atenia_moe_hip_layer_create(desc, &mut raw))?;
        Ok(Self { raw, d_model: desc.d_model as usize })
    }

    pub fn as_raw(&self) -> *mut AteniaMoeLayer {
        self.raw
    }

    /// The op: `[T * d]` in, `[T * d]` out, the whole batch in one call
    /// (`execute_real_moe_layer`, `src/moe/graph_op.rs:327-350`).
    pub fn forward(&self, x: &[f32]) -> Result<Vec<f32>, MoeHipError> {
        if self.d_model == 0 || x.len() % self.d_model != 0 {
            return Err(MoeHipError {
                code: ATENIA_MOE_ERR_DIM,
                message: format!("input length {} is not a multiple of d_model {}", x.len(), self.d_model),
            });
        }
        let mut out = vec![0.0f32; x.len()];
        let t = (x.len() / self.d_model) as c_int;
        check(unsafe { atenia_moe_hip_layer_forward(self.raw, x.as_ptr(), t, out.as_mut_ptr()) })?;
        Ok(out)
    }

    /// (token, expert) of the most recent non-finite routing weight, if any was reported.
    pub fn last_non_finite(&self) -> Option<(i32, i32)> {
        let (mut t, mut e) = (-1i32, -1i32);
        let rc = unsafe { atenia_moe_hip_layer_last_non_finite(self.raw, &mut t, &mut e) };
        if rc == ATENIA_MOE_OK && t >= 0 { Some((t, e)) } else { None }
    }
}

impl Drop for HipMoeLayer {
    fn drop(&mut self) {
        if !self.raw.is_null() {
            unsafe { atenia_moe_hip_layer_destroy(self.raw) };
        }
    }
}
