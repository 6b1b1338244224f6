//! Raw bindings to `libcustos_hip.so`, one declaration per entry point of
//! `include/custos_hip.h` (the counterpart of `src/devices/cuda/api/ffi.rs:165-264` and
//! `src/devices/cuda/api/nvrtc/ffi.rs:36-54`: the library wraps the HIP runtime and hiprtc,
//! so no driver function is bound here).  Every function returns 0 or an error code;
//! `custos_hip_last_error` gives the message.

use core::ffi::{c_char, c_void};

#[repr(C)] pub struct HipDeviceHandle { _p: [u8; 0] }
#[repr(C)] pub struct HipKernel { _p: [u8; 0] }
#[repr(C)] pub struct HipGraph { _p: [u8; 0] }

#[repr(C)]
pub struct HipDeviceInfo {
    pub name: [c_char; 128], pub arch: [c_char; 64], pub compute_units: i32, pub wavefront_size: i32,
    pub clock_khz: i32, pub memory_clock_khz: i32, pub memory_bus_bits: i32, pub l2_bytes: i32,
    pub total_memory: u64,
}
#[repr(C)]
pub struct HipTuning { pub block_threads: i32, pub unroll: i32, pub blocks_per_cu: i32, pub nontemporal: i32, pub direction: i32 }

pub const KIND_APPLY: i32 = 0;
pub const KIND_UNARY_GRAD: i32 = 1;
pub const ALLOC_ZEROED: i32 = 0;
pub const ALLOC_UNINIT: i32 = 1;
pub const LITERALS_ADAPTIVE: i32 = 0;
pub const LITERALS_IN_CODE: i32 = 1;
pub const LITERALS_AS_PARAMETERS: i32 = 2;
pub const GRAPH_EDGES_LEVEL_JOINS: i32 = 0;
pub const GRAPH_EDGES_PER_NODE: i32 = 1;
pub const GRAPH_EDGES_CHAIN: i32 = 2;
pub const GRAPH_EDGES_CHAIN_BY_LEVEL: i32 = 3;

#[link(name = "custos_hip")]
extern "C" {
    pub fn custos_hip_device_count(count: *mut i32) -> i32;
    pub fn custos_hip_device_create(idx: i32, dev: *mut *mut HipDeviceHandle) -> i32;
    pub fn custos_hip_device_destroy(dev: *mut HipDeviceHandle) -> i32;
    pub fn custos_hip_chosen_device_idx() -> i32;
    pub fn custos_hip_get_device_info(dev: *mut HipDeviceHandle, info: *mut HipDeviceInfo) -> i32;
    pub fn custos_hip_last_error(dev: *mut HipDeviceHandle) -> *const c_char;
    pub fn custos_hip_sync(dev: *mut HipDeviceHandle) -> i32;
    pub fn custos_hip_set_tuning(dev: *mut HipDeviceHandle, tuning: *const HipTuning) -> i32;
    pub fn custos_hip_get_tuning(dev: *mut HipDeviceHandle, tuning: *mut HipTuning) -> i32;
    pub fn custos_hip_alloc(dev: *mut HipDeviceHandle, bytes: usize, flags: i32, dptr: *mut u64) -> i32;
    pub fn custos_hip_free(dev: *mut HipDeviceHandle, dptr: u64) -> i32;
    pub fn custos_hip_set_pool_limit(dev: *mut HipDeviceHandle, limit_bytes: usize) -> i32;
    pub fn custos_hip_pool_trim(dev: *mut HipDeviceHandle) -> i32;
    pub fn custos_hip_pool_stats(dev: *mut HipDeviceHandle, pooled_bytes: *mut usize, reused: *mut u64,
                                 allocated: *mut u64) -> i32;
    pub fn custos_hip_write(dev: *mut HipDeviceHandle, dst: u64, src: *const c_void, bytes: usize) -> i32;
    pub fn custos_hip_read(dev: *mut HipDeviceHandle, dst: *mut c_void, src: u64, bytes: usize) -> i32;
    pub fn custos_hip_copy(dev: *mut HipDeviceHandle, dst: u64, src: u64, bytes: usize) -> i32;
    pub fn custos_hip_clear(dev: *mut HipDeviceHandle, dptr: u64, bytes: usize) -> i32;
    pub fn custos_hip_fill(dev: *mut HipDeviceHandle, dptr: u64, bytes: usize, value: *const c_void,
                           value_bytes: usize) -> i32;
    pub fn custos_hip_expr_compile(dev: *mut HipDeviceHandle, kind: i32, dtype: i32, src: *const c_char,
                                   markers: *const *const c_char, n_markers: i32, kernel: *mut *mut HipKernel) -> i32;
    pub fn custos_hip_kernel_source(kernel: *const HipKernel) -> *const c_char;
    pub fn custos_hip_kernel_name(kernel: *const HipKernel) -> *const c_char;
    pub fn custos_hip_kernel_hash(kernel: *const HipKernel) -> u64;
    pub fn custos_hip_kernel_arity(kernel: *const HipKernel) -> i32;
    pub fn custos_hip_kernel_launched_as(dev: *mut HipDeviceHandle, kernel: *mut HipKernel, n: usize,
                                         variant: *mut *mut HipKernel) -> i32;
    pub fn custos_hip_set_literal_policy(dev: *mut HipDeviceHandle, policy: i32) -> i32;
    pub fn custos_hip_launch_hint_stats(dev: *mut HipDeviceHandle, unrelated: *mut u64, resident: *mut u64,
                                        streaming: *mut u64) -> i32;
    pub fn custos_hip_cache_stats(dev: *mut HipDeviceHandle, compiles: *mut u64, hits: *mut u64) -> i32;
    pub fn custos_hip_cache_disk_hits(dev: *mut HipDeviceHandle, disk_hits: *mut u64) -> i32;
    pub fn custos_hip_source_compile(dev: *mut HipDeviceHandle, src: *const c_char, fn_name: *const c_char,
                                     kernel: *mut *mut HipKernel) -> i32;
    pub fn custos_hip_source_launch(dev: *mut HipDeviceHandle, kernel: *mut HipKernel, grid: *const u32,
                                    block: *const u32, shared_mem_bytes: u32, params: *const *mut c_void,
                                    param_sizes: *const usize, n_params: i32) -> i32;
    pub fn custos_hip_source_launch1d(dev: *mut HipDeviceHandle, kernel: *mut HipKernel, len: usize,
                                      params: *const *mut c_void, param_sizes: *const usize, n_params: i32) -> i32;
    pub fn custos_hip_expr_emit(kind: i32, dtype: i32, src: *const c_char, markers: *const *const c_char,
                                n_markers: i32, tuning: *const HipTuning, buf: *mut c_char, cap: usize,
                                needed: *mut usize, hash: *mut u64) -> i32;
    pub fn custos_hip_expr_emit_shared(kind: i32, dtype: i32, src: *const c_char, markers: *const *const c_char,
                                       n_markers: i32, tuning: *const HipTuning, buf: *mut c_char, cap: usize,
                                       needed: *mut usize, hash: *mut u64) -> i32;
    pub fn custos_hip_expr_build_code_object(kind: i32, dtype: i32, src: *const c_char,
                                             markers: *const *const c_char, n_markers: i32,
                                             tuning: *const HipTuning, code_size: *mut usize) -> i32;
    pub fn custos_hip_preferred_shape(footprint_bytes: u64, n_operands: i32, unroll: *mut i32,
                                      nontemporal: *mut i32, alternate: *mut i32) -> i32;
    pub fn custos_hip_preferred_shape_of(footprint_bytes: u64, n_operands: i32, n_written: i32, working_set_bytes: u64,
                                         revisits: i32, unroll: *mut i32, nontemporal: *mut i32, alternate: *mut i32,
                                         block_threads: *mut i32) -> i32;
    pub fn custos_hip_capture_stats(dev: *mut HipDeviceHandle, reused_while_recording: *mut u64, reused_by_comparison: *mut u64,
                                    built: *mut u64) -> i32;
    pub fn custos_hip_check_operand_sets(operands: *const u64, operands_per_set: i32, n_sets: usize, written: i32, bytes: u64) -> i32;
    pub fn custos_hip_set_graph_fusing(dev: *mut HipDeviceHandle, enabled: i32) -> i32;
    pub fn custos_hip_graph_node_kernel(graph: *mut HipGraph, node: usize, name: *mut *const c_char) -> i32;
    pub fn custos_hip_graph_fused_launches(graph: *mut HipGraph, launches: *mut usize) -> i32;
    pub fn custos_hip_chain_emit(dtype: i32, stage_srcs: *const *const c_char, stage_vars: *const i32, n_stages: i32,
                                 sources: *const i32, stage_outs: *const i32, n_inputs: i32, n_outputs: i32,
                                 literals_as_parameters: i32, buf: *mut c_char, cap: usize, needed: *mut usize, code_size: *mut usize) -> i32;
    pub fn custos_hip_last_launch_shape(dev: *mut HipDeviceHandle, unroll: *mut i32, nontemporal: *mut i32,
                                        alternate: *mut i32) -> i32;
    pub fn custos_hip_expr_canonical(src: *const c_char, markers: *const *const c_char, n_markers: i32,
                                     buf: *mut c_char, cap: usize, needed: *mut usize) -> i32;
    pub fn custos_hip_expr_constants(dtype: i32, src: *const c_char, markers: *const *const c_char, n_markers: i32,
                                     buf: *mut c_void, cap: usize, needed: *mut usize, n_params: *mut i32) -> i32;
    pub fn custos_hip_apply_fn(dev: *mut HipDeviceHandle, kernel: *mut HipKernel, x: u64, out: u64, n: usize) -> i32;
    pub fn custos_hip_apply_fn2(dev: *mut HipDeviceHandle, kernel: *mut HipKernel, lhs: u64, rhs: u64, out: u64,
                                n: usize) -> i32;
    pub fn custos_hip_apply_fn_n(dev: *mut HipDeviceHandle, kernel: *mut HipKernel, ins: *const u64, n_ins: i32,
                                 out: u64, n: usize) -> i32;
    pub fn custos_hip_apply_fn_many_noalloc(dev: *mut HipDeviceHandle, kernel: *mut HipKernel, operands: *const u64,
                                            operands_per_set: i32, n_sets: usize, n: usize) -> i32;
    pub fn custos_hip_set_eq_policy(dev: *mut HipDeviceHandle, policy: i32) -> i32;
    pub fn custos_hip_kernel_prepare_merged(dev: *mut HipDeviceHandle, kernel: *mut HipKernel) -> i32;
    pub fn custos_hip_set_graph_fusing_budget(dev: *mut HipDeviceHandle, milliseconds: u32) -> i32;
    pub fn custos_hip_graph_unjoined(graph: *mut HipGraph, launches: *mut usize, reason: *mut *const c_char) -> i32;
    pub fn custos_hip_compile_stats(dev: *mut HipDeviceHandle, units: *mut u64, milliseconds: *mut f64) -> i32;
    pub fn custos_hip_add_unary_grad(dev: *mut HipDeviceHandle, kernel: *mut HipKernel, lhs: u64, lhs_grad: u64,
                                     out_grad: u64, n: usize) -> i32;
    pub fn custos_hip_capture_begin(dev: *mut HipDeviceHandle) -> i32;
    pub fn custos_hip_capture_end(dev: *mut HipDeviceHandle, graph: *mut *mut HipGraph) -> i32;
    pub fn custos_hip_capture_end_reuse(dev: *mut HipDeviceHandle, previous: *mut HipGraph,
                                        graph: *mut *mut HipGraph) -> i32;
    pub fn custos_hip_set_graph_batching(dev: *mut HipDeviceHandle, enabled: i32) -> i32;
    pub fn custos_hip_set_graph_direct_replay(dev: *mut HipDeviceHandle, max_nodes: i32) -> i32;
    pub fn custos_hip_set_graph_edges(dev: *mut HipDeviceHandle, mode: i32) -> i32;
    pub fn custos_hip_set_graph_verify(dev: *mut HipDeviceHandle, enabled: i32) -> i32;
    pub fn custos_hip_graph_edge_count(graph: *mut HipGraph, edges: *mut usize) -> i32;
    pub fn custos_hip_is_capturing(dev: *mut HipDeviceHandle, capturing: *mut i32) -> i32;
    pub fn custos_hip_graph_launch(dev: *mut HipDeviceHandle, graph: *mut HipGraph) -> i32;
    pub fn custos_hip_graph_node_count(graph: *mut HipGraph, kernel_nodes: *mut usize) -> i32;
    pub fn custos_hip_graph_stats(graph: *mut HipGraph, recorded: *mut usize, kernel_nodes: *mut usize,
                                  levels: *mut usize) -> i32;
    pub fn custos_hip_graph_destroy(dev: *mut HipDeviceHandle, graph: *mut HipGraph) -> i32;
    pub fn custos_hip_timer_begin(dev: *mut HipDeviceHandle) -> i32;
    pub fn custos_hip_timer_end(dev: *mut HipDeviceHandle, ms: *mut f64) -> i32;
    pub fn custos_hip_timer_mark(dev: *mut HipDeviceHandle, index: u32) -> i32;
    pub fn custos_hip_timer_between(dev: *mut HipDeviceHandle, first: u32, second: u32, ms: *mut f64) -> i32;
}
