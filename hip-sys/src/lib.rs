//! Rust FFI bindings for `libmonarch_hip.so` (C ABI: `include/monarch_hip.h`).
//!
//! The sibling of the reference's `cuda-sys` / `nccl-sys` crates for the mesh
//! data-movement / reduce path on MI355X: `ndslice::Slice`-described pack/unpack into
//! `RdmaBuffer` staging memory, the local combine of `Communicator::all_reduce` /
//! `reduce_scatter_tensor`, and the block-scaled fp8 codec.  Every function returns a
//! status (`0` = success, `1..9999` = `hipError_t`, `>= 10000` = library classes, see
//! `status` below); device functions enqueue on the given `hipStream_t` and never block.
//!
//! This crate is written against the header by hand (no bindgen) and has not been
//! compiled in the build environment of this repository, which ships no Rust toolchain;
//! `tests/test_abi.py` checks every declaration here against the header, name by name and type by type.
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_int, c_void};

/// `hipStream_t`; replaces `cudaStream_t` of `nccl-sys` on this path.
pub type mhip_stream_t = *mut c_void;
/// `hipEvent_t`.
pub type mhip_event_t = *mut c_void;

/// `ndslice::Slice` as the C ABI sees it: `sizes`/`strides` point at `ndim` `usize`s
/// (`Slice::sizes().as_ptr()` / `Slice::strides().as_ptr()` on a 64-bit target).
#[repr(C)]
#[derive(Debug, Clone, Copy)]
pub struct mhip_slice_t {
    pub offset: u64,
    pub ndim: u32,
    pub sizes: *const u64,
    pub strides: *const u64,
}

/// `monarch_rdma::RdmaBuffer` without its NIC fields: `{addr, size}` of a registered byte range.
#[repr(C)]
#[derive(Debug, Clone, Copy)]
pub struct mhip_rdma_buffer_t {
    pub addr: *mut c_void,
    pub size: usize,
}

/// `rdmaxcel_sys::wqe_params_t` (`rdmaxcel-sys/src/rdmaxcel.h:26-39`): same fields, order and widths.
#[repr(C)]
#[derive(Debug, Clone, Copy)]
pub struct mhip_wqe_params_t {
    pub laddr: usize,
    pub lkey: u32,
    pub length: usize,
    pub wr_id: u64,
    pub signaled: bool,
    pub op_type: u32,
    pub raddr: usize,
    pub rkey: u32,
    pub qp_num: u32,
    pub buf: *mut u8,
    pub dbrec: *mut u32,
    pub wqe_cnt: u32,
}

/// `rdmaxcel_sys::cqe_poll_params_t` (`rdmaxcel.h:42-48`).
#[repr(C)]
#[derive(Debug, Clone, Copy)]
pub struct mhip_cqe_poll_params_t {
    pub cqe_buf: *mut u8,
    pub cqe_size: u32,
    pub consumer_index: u32,
    pub cqe_cnt: u32,
    pub dbrec: *mut u32,
}

/// `MLX5_OPCODE_*` as `RdmaQueuePair::send_wqe` uses them (`monarch_rdma/src/rdma_components.rs:1119-1124`).
pub const MHIP_MLX5_OPCODE_RDMA_WRITE: u32 = 0x08;
pub const MHIP_MLX5_OPCODE_RDMA_WRITE_IMM: u32 = 0x09;
pub const MHIP_MLX5_OPCODE_RDMA_READ: u32 = 0x10;

/// `Option::None` of `WorkerActor::send_tensor`'s `from_rank` / `to_rank`.
pub const MHIP_NO_RANK: u64 = u64::MAX;

pub mod status {
    pub const SUCCESS: i32 = 0;
    pub const INVALID_DIMS: i32 = 10001;
    pub const NONRECTANGULAR_SHAPE: i32 = 10002;
    pub const NONUNIQUE_STRIDES: i32 = 10003;
    pub const STRIDE_TOO_SMALL: i32 = 10004;
    pub const INDEX_OUT_OF_RANGE: i32 = 10005;
    pub const VALUE_NOT_IN_SLICE: i32 = 10006;
    pub const INCOMPATIBLE_VIEW: i32 = 10007;
    pub const NONCONTIGUOUS: i32 = 10008;
    pub const EMPTY_RANGE: i32 = 10009;
    pub const DIMENSION_OUT_OF_RANGE: i32 = 10010;
    pub const INVALID_DATA_TYPE: i32 = 10101;
    pub const NONCONTIGUOUS_TENSOR: i32 = 10102;
    pub const INVALID_DEVICE: i32 = 10103;
    pub const FLOAT8_REDUCTION: i32 = 10104;
    pub const TYPE_MISMATCH: i32 = 10105;
    pub const OUTPUT_SIZE_MISMATCH: i32 = 10106;
    pub const INPUT_SIZE_MISMATCH: i32 = 10107;
    pub const UNDEFINED_TENSOR: i32 = 10108;
    pub const INVALID_ARGUMENT: i32 = 10201;
    pub const UNSUPPORTED_OP: i32 = 10202;
    pub const TOO_MANY_INPUTS: i32 = 10203;
    pub const UNSUPPORTED_BLOCK: i32 = 10204;
    pub const BUFFER_TOO_SMALL: i32 = 10205;
    pub const SCRATCH_TOO_SMALL: i32 = 10206;
    pub const WQE_OVERFLOW: i32 = 10207;
    pub const MESH_DIM_LENGTH_MISMATCH: i32 = 10301;
    pub const MESH_DIM_MISSING: i32 = 10302;
}

/// `c10::ScalarType` numbering, as carried by `monarch_messages::worker::Factory::dtype`.
pub mod dtype {
    pub const U8: i32 = 0;
    pub const I8: i32 = 1;
    pub const I32: i32 = 3;
    pub const I64: i32 = 4;
    pub const F16: i32 = 5;
    pub const F32: i32 = 6;
    pub const F64: i32 = 7;
    pub const BF16: i32 = 15;
    pub const F8E5M2: i32 = 23;
    pub const F8E4M3FN: i32 = 24;
    pub const F8E5M2FNUZ: i32 = 25;
    pub const F8E4M3FNUZ: i32 = 26;
}

/// `ncclRedOp_t` numbering (`torch_sys_cuda::nccl::ReduceOp as i32`).
pub mod op {
    pub const SUM: i32 = 0;
    pub const PROD: i32 = 1;
    pub const MAX: i32 = 2;
    pub const MIN: i32 = 3;
    pub const AVG: i32 = 4;
}

extern "C" {
    pub fn mhip_error_string(status: c_int) -> *const c_char;
    pub fn mhip_version() -> c_int;
    pub fn mhip_dtype_size(dtype: c_int) -> u32;
    pub fn mhip_slice_validate(offset: u64, sizes: *const u64, nsizes: u32, strides: *const u64, nstrides: u32) -> c_int;
    pub fn mhip_slice_len(s: *const mhip_slice_t, len: *mut u64) -> c_int;
    pub fn mhip_slice_is_contiguous(s: *const mhip_slice_t, result: *mut c_int) -> c_int;
    pub fn mhip_slice_get(s: *const mhip_slice_t, index: u64, loc: *mut u64) -> c_int;
    pub fn mhip_slice_location(s: *const mhip_slice_t, coord: *const u64, ncoord: u32, loc: *mut u64) -> c_int;
    pub fn mhip_slice_coordinates(s: *const mhip_slice_t, value: u64, coords: *mut u64) -> c_int;
    pub fn mhip_slice_index(s: *const mhip_slice_t, value: u64, index: *mut u64) -> c_int;
    pub fn mhip_slice_iter(s: *const mhip_slice_t, start: u64, count: u64, locs: *mut u64, written: *mut u64) -> c_int;
    pub fn mhip_slice_select(s: *const mhip_slice_t, dim: u32, begin: u64, end: u64, step: u64, out_offset: *mut u64, out_sizes: *mut u64, out_strides: *mut u64) -> c_int;
    pub fn mhip_slice_at(s: *const mhip_slice_t, dim: u32, index: u64, out_offset: *mut u64, out_sizes: *mut u64, out_strides: *mut u64) -> c_int;
    pub fn mhip_slice_subview(s: *const mhip_slice_t, starts: *const u64, nstarts: u32, lens: *const u64, nlens: u32, out_offset: *mut u64) -> c_int;
    pub fn mhip_slice_view(s: *const mhip_slice_t, new_sizes: *const u64, nnew: u32, out_strides: *mut u64) -> c_int;
    pub fn mhip_slice_enforce_embedding(s: *const mhip_slice_t, other: *const mhip_slice_t) -> c_int;
    pub fn mhip_slice_bounds(s: *const mhip_slice_t, min_loc: *mut u64, max_loc: *mut u64) -> c_int;
    pub fn mhip_mesh_dim_members(ranks: *const mhip_slice_t, rank: u64, dim: u32, members: *mut u64, dim_rank: *mut u64) -> c_int;
    pub fn mhip_mesh_ranks_for_dims(ranks: *const mhip_slice_t, rank: u64, dims: *const u32, ndims: u32, out: *mut u64, cap: u64, count: *mut u64) -> c_int;
    pub fn mhip_slice_pack(dst: *mut c_void, src_base: *const c_void, s: *const mhip_slice_t, elem_size: u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_slice_unpack(dst_base: *mut c_void, src: *const c_void, s: *const mhip_slice_t, elem_size: u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_slice_pack_many(dsts: *const *mut c_void, src_base: *const c_void, views: *const mhip_slice_t, nviews: u32, elem_size: u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_slice_unpack_many(dst_base: *mut c_void, srcs: *const *const c_void, views: *const mhip_slice_t, nviews: u32, elem_size: u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_flat_pack(flat: *mut c_void, d_tensors: *const *const c_void, d_offsets: *const u64, ntensors: u32, total: u64, elem_size: u32, d_index: *const u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_flat_unpack(d_tensors: *const *mut c_void, flat: *const c_void, d_offsets: *const u64, ntensors: u32, total: u64, elem_size: u32, d_index: *const u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_reduce(out: *mut c_void, input: *const *const c_void, n: u32, numel: u64, dtype: c_int, op: c_int, stream: mhip_stream_t) -> c_int;
    pub fn mhip_reduce_scatter(outs: *const *mut c_void, out_views: *const mhip_slice_t, n_out: u32, input: *const *const c_void, in_view: *const mhip_slice_t, in_numel: u64, n_in: u32, dtype: c_int, op: c_int, stream: mhip_stream_t) -> c_int;
    pub fn mhip_stack(out: *mut c_void, input: *const *const c_void, n: u32, numel: u64, elem_size: u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_stack_scatter(out: *mut c_void, input: *const *const c_void, n: u32, rank: u32, numel: u64, elem_size: u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_buffer_read_into(local: *const mhip_rdma_buffer_t, remote: *const mhip_rdma_buffer_t, stream: mhip_stream_t) -> c_int;
    pub fn mhip_buffer_write_from(local: *const mhip_rdma_buffer_t, remote: *const mhip_rdma_buffer_t, stream: mhip_stream_t) -> c_int;
    pub fn mhip_buffer_transfer(dst: *mut c_void, src: *const c_void, bytes: usize, max_segment_bytes: usize, stream: mhip_stream_t, segments: *mut u32) -> c_int;
    pub fn mhip_buffer_transfer_many(dsts: *const *mut c_void, srcs: *const *const c_void, bytes: *const usize, n: u32, max_segment_bytes: usize, stream: mhip_stream_t, segments: *mut u32) -> c_int;
    pub fn mhip_send_tensor_route(from_ranks: *const mhip_slice_t, to_ranks: *const mhip_slice_t, rank: u64, from_rank: *mut u64, to_rank: *mut u64) -> c_int;
    pub fn mhip_to_mesh_from_ranks(slicing_names: *const *const c_char, slicing: *const mhip_slice_t, mesh_names: *const *const c_char, mesh_sizes: *const u64, mesh_ndim: u32, out_sizes: *mut u64, out_strides: *mut u64, out_ndim: *mut u32, broadcast_dims: *mut u32, n_broadcast: *mut u32, culprit: *mut u32) -> c_int;
    pub fn mhip_send_tensor(result: *mut c_void, result_bytes: usize, src_base: *const c_void, src_view: *const mhip_slice_t, elem_size: u32, staging: *mut c_void, stream: mhip_stream_t) -> c_int;
    pub fn mhip_rdmaxcel_send_wqe(params: *const mhip_wqe_params_t, stream: mhip_stream_t) -> c_int;
    pub fn mhip_rdmaxcel_recv_wqe(params: *const mhip_wqe_params_t, stream: mhip_stream_t) -> c_int;
    pub fn mhip_rdmaxcel_db_ring(dst: *mut c_void, src: *const c_void, stream: mhip_stream_t) -> c_int;
    pub fn mhip_rdmaxcel_ring_doorbells(dst: *mut c_void, sq_buf: *const c_void, stride: u32, wqe_cnt: u32, first_db_idx: u32, count: u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_rdmaxcel_cqe_poll(d_result: *mut i32, params: *const mhip_cqe_poll_params_t, stream: mhip_stream_t) -> c_int;
    pub fn mhip_rdmaxcel_post_transfer(params: *const mhip_wqe_params_t, max_segment_bytes: usize, n_wqes: *mut u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_rdmaxcel_send_wqe_host(params: *const mhip_wqe_params_t) -> c_int;
    pub fn mhip_rdmaxcel_recv_wqe_host(params: *const mhip_wqe_params_t) -> c_int;
    pub fn mhip_rdmaxcel_db_ring_host(dst: *mut c_void, src: *const c_void) -> c_int;
    pub fn mhip_rdmaxcel_cqe_poll_host(result: *mut i32, params: *const mhip_cqe_poll_params_t) -> c_int;
    pub fn mhip_fp8_quantize(q: *mut u8, scales: *mut f32, x_bf16: *const c_void, numel: u64, block: u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_fp8_dequant_accumulate(acc: *mut f32, q: *const u8, scales: *const f32, numel: u64, block: u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_fp8_dequant_accumulate_many(acc: *mut f32, q: *const *const u8, scales: *const *const f32, n: u32, numel: u64, block: u32, overwrite: c_int, stream: mhip_stream_t) -> c_int;
    pub fn mhip_fp8_quantize_bucket(q: *mut u8, scales: *mut f32, d_tensors: *const *const c_void, d_offsets: *const u64, ntensors: u32, total: u64, block: u32, d_index: *const u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_fp8_dequant_accumulate_bucket(d_acc_tensors: *const *mut c_void, q: *const u8, scales: *const f32, d_offsets: *const u64, ntensors: u32, total: u64, block: u32, d_index: *const u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_fp8_dequant_accumulate_bucket_many(d_acc_tensors: *const *mut c_void, q: *const *const u8, scales: *const *const f32, n: u32, d_offsets: *const u64, ntensors: u32, total: u64, block: u32, d_index: *const u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_fp8_quantize_bucket_static(q: *mut u8, scales: *mut f32, d_tensors: *const *const c_void, d_offsets: *const u64, ntensors: u32, total: u64, block: u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_bucket_index_bytes(total: u64, block: u32, bytes: *mut usize) -> c_int;
    pub fn mhip_bucket_index_build(d_index: *mut u32, d_offsets: *const u64, ntensors: u32, total: u64, block: u32, stream: mhip_stream_t) -> c_int;
    pub fn mhip_device_count(count: *mut c_int) -> c_int;
    pub fn mhip_set_device(device: c_int) -> c_int;
    pub fn mhip_device_synchronize() -> c_int;
    pub fn mhip_stream_create(stream: *mut mhip_stream_t) -> c_int;
    pub fn mhip_stream_destroy(stream: mhip_stream_t) -> c_int;
    pub fn mhip_stream_synchronize(stream: mhip_stream_t) -> c_int;
    pub fn mhip_event_create(event: *mut mhip_event_t) -> c_int;
    pub fn mhip_event_destroy(event: mhip_event_t) -> c_int;
    pub fn mhip_event_record(event: mhip_event_t, stream: mhip_stream_t) -> c_int;
    pub fn mhip_event_synchronize(event: mhip_event_t) -> c_int;
    pub fn mhip_event_elapsed_ms(ms: *mut f32, start: mhip_event_t, stop: mhip_event_t) -> c_int;
    pub fn mhip_stream_wait_event(stream: mhip_stream_t, event: mhip_event_t) -> c_int;
    pub fn mhip_malloc(ptr: *mut *mut c_void, bytes: usize) -> c_int;
    pub fn mhip_free(ptr: *mut c_void) -> c_int;
    pub fn mhip_memcpy_htod(dst: *mut c_void, src: *const c_void, bytes: usize, stream: mhip_stream_t) -> c_int;
    pub fn mhip_memcpy_dtoh(dst: *mut c_void, src: *const c_void, bytes: usize, stream: mhip_stream_t) -> c_int;
    pub fn mhip_memset(dst: *mut c_void, value: c_int, bytes: usize, stream: mhip_stream_t) -> c_int;
    pub fn mhip_staging_alloc(ptr: *mut *mut c_void, padded_bytes: *mut usize, bytes: usize, device: c_int) -> c_int;
    pub fn mhip_staging_free(ptr: *mut c_void, padded_bytes: usize) -> c_int;
    pub fn mhip_staging_slot_pitch(slot_bytes: usize, pitch_bytes: *mut usize) -> c_int;
    pub fn mhip_pointer_is_device(ptr: *const c_void, is_device: *mut c_int) -> c_int;
    pub fn mhip_export_dmabuf(fd: *mut c_int, ptr: *const c_void, bytes: usize) -> c_int;
}

#[cfg(test)]
mod tests {
    use super::*;

    #[test]
    fn sanity() {
        // SAFETY: testing bindings; host-only calls, no GPU needed
        unsafe {
            assert!(mhip_version() >= 100);
            let sizes = [2u64, 3];
            let strides = [3u64, 1];
            assert_eq!(mhip_slice_validate(0, sizes.as_ptr(), 2, strides.as_ptr(), 2), status::SUCCESS);
            let s = mhip_slice_t { offset: 0, ndim: 2, sizes: sizes.as_ptr(), strides: strides.as_ptr() };
            let mut loc = 0u64;
            assert_eq!(mhip_slice_get(&s, 4, &mut loc), status::SUCCESS);
            assert_eq!(loc, 4);
        }
    }
}
