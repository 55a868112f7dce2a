/*
 * monarch_hip.h - C ABI of libmonarch_hip.so: the MI355X (gfx950) data plane for
 * Monarch's mesh data-movement / reduce path.
 *
 * This is the contract a `hip-sys` crate binds (the sibling of the reference's
 * cuda-sys/ and nccl-sys/ crates).  Plain pointers and sizes only; every entry
 * point returns an int status (0 = success, 1..9999 = hipError_t passed through,
 * >= 10000 = the library's own classes below).  Device entry points enqueue on the
 * caller's stream and never synchronise; completion is observed the way the
 * reference does it, by recording an event on that stream afterwards
 * (monarch_tensor_worker/src/comm.rs:156).  All device pointers are caller-owned:
 * no data-path entry point allocates or frees device memory (the only allocating
 * calls are the explicit mhip_staging_alloc, mhip_stream_create and mhip_event_create
 * near the end of this file).  Entry points may be called from any thread; the
 * device is taken from the stream (or is the current device for the NULL stream).
 *
 * Units: a Slice counts ELEMENTS (ndslice/src/slice.rs:85-90); pack/unpack take the
 * element size in bytes; RdmaBuffer-style staging memory is addressed in bytes
 * (monarch_rdma/src/rdma_components.rs:94-102).
 */
#ifndef MONARCH_HIP_H
#define MONARCH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* hipStream_t / hipEvent_t, kept opaque so that binding this header needs no HIP headers.
 * Replaces cudaStream_t / CUstream_st of nccl-sys/build.rs:93-148 and
 * torch-sys-cuda/src/cuda.rs:15-17 on this path. */
typedef void* mhip_stream_t;
typedef void* mhip_event_t;

/* ---- status codes ---- */
enum {
    MHIP_SUCCESS = 0,
    /* SliceError, ndslice/src/slice.rs:15-51 */
    MHIP_ERR_INVALID_DIMS = 10001,
    MHIP_ERR_NONRECTANGULAR_SHAPE = 10002,
    MHIP_ERR_NONUNIQUE_STRIDES = 10003,
    MHIP_ERR_STRIDE_TOO_SMALL = 10004,
    MHIP_ERR_INDEX_OUT_OF_RANGE = 10005,
    MHIP_ERR_VALUE_NOT_IN_SLICE = 10006,
    MHIP_ERR_INCOMPATIBLE_VIEW = 10007,
    MHIP_ERR_NONCONTIGUOUS = 10008,
    MHIP_ERR_EMPTY_RANGE = 10009,
    MHIP_ERR_DIMENSION_OUT_OF_RANGE = 10010,
    /* NcclError argument checks, torch-sys-cuda/src/nccl.rs:56-93 */
    MHIP_ERR_INVALID_DATA_TYPE = 10101,
    MHIP_ERR_NONCONTIGUOUS_TENSOR = 10102,
    MHIP_ERR_INVALID_DEVICE = 10103,
    MHIP_ERR_FLOAT8_REDUCTION = 10104,
    MHIP_ERR_TYPE_MISMATCH = 10105,
    MHIP_ERR_OUTPUT_SIZE_MISMATCH = 10106,
    MHIP_ERR_INPUT_SIZE_MISMATCH = 10107,
    MHIP_ERR_UNDEFINED_TENSOR = 10108,
    /* library-specific */
    MHIP_ERR_INVALID_ARGUMENT = 10201,
    MHIP_ERR_UNSUPPORTED_OP = 10202,
    MHIP_ERR_TOO_MANY_INPUTS = 10203,
    MHIP_ERR_UNSUPPORTED_BLOCK = 10204,
    MHIP_ERR_BUFFER_TOO_SMALL = 10205,
    MHIP_ERR_SCRATCH_TOO_SMALL = 10206,
    MHIP_ERR_WQE_OVERFLOW = 10207,
    /* Tensor.to_mesh checks, python/monarch/common/tensor.py:426-437 */
    MHIP_ERR_MESH_DIM_LENGTH_MISMATCH = 10301,
    MHIP_ERR_MESH_DIM_MISSING = 10302
};

/* Text for any status this library returns (hipGetErrorString for HIP codes);
 * the counterpart of cuGetErrorString in monarch_rdma/src/macros.rs:9-24. */
const char* mhip_error_string(int status);
/* Library version, major*10000 + minor*100 + patch. */
int mhip_version(void);

/* ---- element types: c10::ScalarType numbering, as carried by
 * monarch_messages Factory.dtype (monarch_messages/src/worker.rs:434-447) ---- */
enum {
    MHIP_DTYPE_U8 = 0,
    MHIP_DTYPE_I8 = 1,
    MHIP_DTYPE_I32 = 3,
    MHIP_DTYPE_I64 = 4,
    MHIP_DTYPE_F16 = 5,
    MHIP_DTYPE_F32 = 6,
    MHIP_DTYPE_F64 = 7,
    MHIP_DTYPE_BF16 = 15,
    MHIP_DTYPE_F8E5M2 = 23,
    MHIP_DTYPE_F8E4M3FN = 24,
    MHIP_DTYPE_F8E5M2FNUZ = 25,
    MHIP_DTYPE_F8E4M3FNUZ = 26
};
/* Size in bytes of a dtype, 0 if unknown. */
uint32_t mhip_dtype_size(int dtype);

/* ncclRedOp_t numbering, torch-sys-cuda/src/nccl.rs:285-292. */
enum { MHIP_OP_SUM = 0, MHIP_OP_PROD = 1, MHIP_OP_MAX = 2, MHIP_OP_MIN = 3, MHIP_OP_AVG = 4 };

/* ====================================================================== */
/* Slice: host-side index algebra (no GPU needed)                         */
/* ====================================================================== */

/* ndslice::Slice {offset, sizes, strides}, ndslice/src/slice.rs:85-90.  sizes and
 * strides each hold ndim entries and stay owned by the caller. */
typedef struct {
    uint64_t offset;
    uint32_t ndim;
    const uint64_t* sizes;
    const uint64_t* strides;
} mhip_slice_t;

#define MHIP_MAX_DIMS 32

/* Slice::new validation (slice.rs:99-139): same rules, same error classes, same order. */
int mhip_slice_validate(uint64_t offset, const uint64_t* sizes, uint32_t nsizes,
                        const uint64_t* strides, uint32_t nstrides);
/* Slice::len (slice.rs:382-384). */
int mhip_slice_len(const mhip_slice_t* s, uint64_t* len);
/* Slice::is_contiguous (slice.rs:198-207). */
int mhip_slice_is_contiguous(const mhip_slice_t* s, int* result);
/* Slice::get (slice.rs:523-537). */
int mhip_slice_get(const mhip_slice_t* s, uint64_t index, uint64_t* loc);
/* Slice::location (slice.rs:330-343). */
int mhip_slice_location(const mhip_slice_t* s, const uint64_t* coord, uint32_t ncoord, uint64_t* loc);
/* Slice::coordinates (slice.rs:347-374); coords holds ndim entries. */
int mhip_slice_coordinates(const mhip_slice_t* s, uint64_t value, uint64_t* coords);
/* Slice::index (slice.rs:460-471). */
int mhip_slice_index(const mhip_slice_t* s, uint64_t value, uint64_t* index);
/* Slice::iter (slice.rs:391-396, 704-781): locations of items [start, start+count) of the
 * row-major enumeration, clipped to len; *written receives how many were produced. */
int mhip_slice_iter(const mhip_slice_t* s, uint64_t start, uint64_t count, uint64_t* locs,
                    uint64_t* written);
/* Slice::select (slice.rs:291-327); out arrays hold ndim entries. */
int mhip_slice_select(const mhip_slice_t* s, uint32_t dim, uint64_t begin, uint64_t end,
                      uint64_t step, uint64_t* out_offset, uint64_t* out_sizes,
                      uint64_t* out_strides);
/* Slice::at (slice.rs:243-264); out arrays hold ndim-1 entries. */
int mhip_slice_at(const mhip_slice_t* s, uint32_t dim, uint64_t index, uint64_t* out_offset,
                  uint64_t* out_sizes, uint64_t* out_strides);
/* Slice::subview (slice.rs:638-661): result is {*out_offset, lens, s->strides}. */
int mhip_slice_subview(const mhip_slice_t* s, const uint64_t* starts, uint32_t nstarts,
                       const uint64_t* lens, uint32_t nlens, uint64_t* out_offset);
/* Slice::view (slice.rs:579-635): result is {0, new_sizes, out_strides}. */
int mhip_slice_view(const mhip_slice_t* s, const uint64_t* new_sizes, uint32_t nnew,
                    uint64_t* out_strides);
/* Slice::enforce_embedding (slice.rs:683-687). */
int mhip_slice_enforce_embedding(const mhip_slice_t* s, const mhip_slice_t* other);
/* Smallest and largest location the slice touches (for sizing/guarding the base
 * allocation); MHIP_ERR_INVALID_ARGUMENT for an empty slice.  No reference counterpart. */
int mhip_slice_bounds(const mhip_slice_t* s, uint64_t* min_loc, uint64_t* max_loc);

/* DeviceMesh::new, one dimension (monarch_tensor_worker/src/device_mesh.rs:71-102):
 * members[0..sizes[dim]) and the owning rank's position among them. */
int mhip_mesh_dim_members(const mhip_slice_t* ranks, uint64_t rank, uint32_t dim,
                          uint64_t* members, uint64_t* dim_rank);
/* DeviceMesh::get_ranks_for_dim_slice (device_mesh.rs:120-177): the reduce group of the
 * named dims (given as dim indices, in the caller's order); *count receives the group
 * size N that Avg divides by and scatter splits into (monarch_tensor_worker/src/lib.rs:899,911). */
int mhip_mesh_ranks_for_dims(const mhip_slice_t* ranks, uint64_t rank, const uint32_t* dims,
                             uint32_t ndims, uint64_t* out, uint64_t cap, uint64_t* count);

/* ====================================================================== */
/* pack / unpack: Slice view <-> contiguous staging memory                 */
/* ====================================================================== */

/* dst[i] = src_base[s.get(i)] for i in [0, len): gathers the view, in Slice::iter order
 * (slice.rs:391-396), into contiguous staging memory - the bytes an RdmaBuffer
 * {addr = dst, size = len*elem_size} then moves with read_into
 * (monarch_rdma/src/rdma_components.rs:117-137).  The slice must pass mhip_slice_validate.
 * dst must not overlap the view. */
int mhip_slice_pack(void* dst, const void* src_base, const mhip_slice_t* s, uint32_t elem_size,
                    mhip_stream_t stream);
/* dst_base[s.get(i)] = src[i]: scatters staging memory that write_from filled
 * (rdma_components.rs:152-171) back into the view; elements outside the view are untouched. */
int mhip_slice_unpack(void* dst_base, const void* src, const mhip_slice_t* s, uint32_t elem_size,
                      mhip_stream_t stream);
/* nviews packs / unpacks of views of ONE base tensor in a single launch (a reshard's
 * column blocks): dsts[k][i] = src_base[views[k].get(i)], resp. the inverse. */
int mhip_slice_pack_many(void* const* dsts, const void* src_base, const mhip_slice_t* views,
                         uint32_t nviews, uint32_t elem_size, mhip_stream_t stream);
int mhip_slice_unpack_many(void* dst_base, const void* const* srcs, const mhip_slice_t* views,
                           uint32_t nviews, uint32_t elem_size, mhip_stream_t stream);

/* Flat bucket with an offsets table (torch.cat / split of a gradient bucket,
 * python/tests/simulator/test_simulator.py:190-203, for ragged tensors):
 * flat[offsets[t] + j] = tensors[t][j].  d_tensors (ntensors pointers) and d_offsets
 * (ntensors+1 element offsets, offsets[0] == 0) live in DEVICE memory; total ==
 * offsets[ntensors] is passed by value so that the call needs no device read-back.
 * d_index: the bucket's block index written by mhip_bucket_index_build (below), or NULL.
 * With it a wavefront finds its tensor with one load instead of a table search and the copy
 * runs as single-wavefront workgroups; the bytes moved are the same either way. */
int mhip_flat_pack(void* flat, const void* const* d_tensors, const uint64_t* d_offsets,
                   uint32_t ntensors, uint64_t total, uint32_t elem_size, const uint32_t* d_index,
                   mhip_stream_t stream);
int mhip_flat_unpack(void* const* d_tensors, const void* flat, const uint64_t* d_offsets,
                     uint32_t ntensors, uint64_t total, uint32_t elem_size, const uint32_t* d_index,
                     mhip_stream_t stream);

/* ====================================================================== */
/* Reduce: the chunks one GPU owns                                         */
/* ====================================================================== */

/* out[i] = op_r in[r][i], r in [0, n): the local combine of Communicator::all_reduce
 * (torch-sys-cuda/src/nccl.rs:464-489) as StreamActor::reduce uses it
 * (monarch_tensor_worker/src/stream.rs:1437-1462).  out may coincide with exactly one of
 * the inputs (the in-place form); any other overlap is undefined.  Floating types accumulate in fp32 (f64 in f64)
 * in rank order and round once; Avg divides the sum by n.  Integer Sum and Prod wrap.
 * Max / Min keep the accumulator on ties and skip NaN operands unless all are NaN (fmaxf / fminf,
 * which is how NCCL's own kernels define ncclMax / ncclMin; NCCL is outside the reference tree);
 * I8 / I32 / I64 compare as signed, U8 as unsigned.
 * Argument checks follow nccl.rs:300-316,474-476: null pointer -> UNDEFINED_TENSOR,
 * unknown dtype -> INVALID_DATA_TYPE, fp8 dtype -> FLOAT8_REDUCTION; an op outside
 * nccl.rs:285-292, or Avg on an integer dtype -> UNSUPPORTED_OP; n > 64 -> TOO_MANY_INPUTS. */
int mhip_reduce(void* out, const void* const* in, uint32_t n, uint64_t numel, int dtype, int op,
                mhip_stream_t stream);

/* reduced[i] = op_g in[g][in_view.get(i)] over in_view's index space;
 * outs[k][j] = reduced[out_views[k].get(j)]: the local combine of
 * Communicator::reduce_scatter_tensor (nccl.rs:661-703; stream.rs:1422-1436) with the
 * scatter expressed as Slice views of the reduced tensor.  in_view == NULL means the
 * n_in inputs are contiguous with len == in_numel.  ncclReduceScatter's flat-chunk rule
 * is out_views[k] = {k*c, [c], [1]}.  outs must not alias the inputs (scatter is never in
 * place, stream.rs:1423). */
int mhip_reduce_scatter(void* const* outs, const mhip_slice_t* out_views, uint32_t n_out,
                        const void* const* in, const mhip_slice_t* in_view, uint64_t in_numel,
                        uint32_t n_in, int dtype, int op, mhip_stream_t stream);

/* Reduction::Stack without scatter: the data movement of Communicator::all_gather_into_tensor as
 * StreamActor::reduce uses it (monarch_tensor_worker/src/stream.rs:1408-1417; result shape
 * [n, *factory.size], the reference's test is torch-sys-cuda/src/nccl.rs:927-959):
 * out[g * numel + i] = in[g][i] for the n <= 64 members' tensors, in one launch.  out must not
 * overlap an input. */
int mhip_stack(void* out, const void* const* in, uint32_t n, uint64_t numel, uint32_t elem_size,
               mhip_stream_t stream);
/* Reduction::Stack with scatter: Communicator::all_to_all_single (nccl.rs:760-812; stream.rs:1381-1399)
 * as member `rank` sees it, every member's tensor holding numel elements cut into n equal chunks of
 * c = numel / n:  out[g * c + i] = in[g][rank * c + i].  numel % n != 0 -> INPUT_SIZE_MISMATCH.
 * out may be in[rank] (the in-place form); chunks g != rank of that tensor are then overwritten. */
int mhip_stack_scatter(void* out, const void* const* in, uint32_t n, uint32_t rank, uint64_t numel,
                       uint32_t elem_size, mhip_stream_t stream);

/* ====================================================================== */
/* RdmaBuffer transfers and SendTensor                                     */
/* ====================================================================== */

/* RdmaBuffer (monarch_rdma/src/rdma_components.rs:94-102) without its NIC fields (owner, mr_id,
 * lkey, rkey): a contiguous registered byte range.  Owns nothing. */
typedef struct {
    void* addr;
    size_t size;
} mhip_rdma_buffer_t;

/* local.read_into(remote), rdma_components.rs:117-137 -> RdmaQueuePair::put (:842-858): local.size bytes
 * go from local.addr to remote.addr.  On one GPU the transport is a device copy on `stream`, posted as
 * one copy per work request: a request's length is a 32-bit field (rdma_components.rs:1041,1063), so
 * transfers are cut into requests of at most 2^32 - 16 bytes instead of being truncated.
 * local.size > remote.size -> BUFFER_TOO_SMALL (a NIC refuses a write past the remote region). */
int mhip_buffer_read_into(const mhip_rdma_buffer_t* local, const mhip_rdma_buffer_t* remote,
                          mhip_stream_t stream);
/* local.write_from(remote), rdma_components.rs:152-171 -> RdmaQueuePair::get (:986-1002): local.size
 * bytes go from remote.addr to local.addr. */
int mhip_buffer_write_from(const mhip_rdma_buffer_t* local, const mhip_rdma_buffer_t* remote,
                           mhip_stream_t stream);
/* The request walk both calls share: `bytes` bytes from src to dst in requests of at most
 * max_segment_bytes (0, or anything above it, means the wire limit of 2^32 - 16); *segments, when not
 * NULL, receives the number of requests posted. */
int mhip_buffer_transfer(void* dst, const void* src, size_t bytes, size_t max_segment_bytes,
                         mhip_stream_t stream, uint32_t* segments);
/* n such transfers, bytes[g] bytes from srcs[g] to dsts[g], with the requests of all of them in one launch
 * (64 requests per launch): a message that moves several staging buffers, such as the column blocks
 * of a reshard, pays for one launch instead of n.  The reference posts its work requests one by one
 * (rdma_components.rs:842-858, :986-1002), so this has no single counterpart there; the bytes moved are
 * those of n mhip_buffer_transfer calls.  Buffers must not overlap each other. */
int mhip_buffer_transfer_many(void* const* dsts, const void* const* srcs, const size_t* bytes, uint32_t n,
                              size_t max_segment_bytes, mhip_stream_t stream, uint32_t* segments);

#define MHIP_NO_RANK UINT64_MAX
/* WorkerActor::send_tensor's routing (monarch_tensor_worker/src/lib.rs:722-731): the i-th rank of
 * from_ranks sends to the i-th rank of to_ranks.  *to_rank = to_ranks.get(from_ranks.index(rank)),
 * *from_rank = from_ranks.get(to_ranks.index(rank)), each MHIP_NO_RANK when `rank` is not in the
 * respective slice (Option::None in the reference). */
int mhip_send_tensor_route(const mhip_slice_t* from_ranks, const mhip_slice_t* to_ranks, uint64_t rank,
                           uint64_t* from_rank, uint64_t* to_rank);
/* Tensor.to_mesh's client-side check (python/monarch/common/tensor.py:417-438): for every dimension
 * of the destination mesh (names and sizes, in mesh order) that the source slicing names, its size
 * must match; the from_ranks slice is {slicing.offset, out_sizes, out_strides} with *out_ndim entries;
 * destination dimensions the slicing does not name are broadcast dimensions (indices into the mesh).
 * Errors: MESH_DIM_LENGTH_MISMATCH (*culprit = the mesh dimension), MESH_DIM_MISSING (*culprit = the
 * first slicing dimension the destination lacks).  out_sizes / out_strides hold slicing->ndim
 * entries, broadcast_dims mesh_ndim entries; culprit may be NULL. */
int mhip_to_mesh_from_ranks(const char* const* slicing_names, const mhip_slice_t* slicing,
                            const char* const* mesh_names, const uint64_t* mesh_sizes,
                            uint32_t mesh_ndim, uint64_t* out_sizes, uint64_t* out_strides,
                            uint32_t* out_ndim, uint32_t* broadcast_dims, uint32_t* n_broadcast,
                            uint32_t* culprit);
/* StreamActor::send_tensor (monarch_tensor_worker/src/stream.rs:1470-1560) for data on one GPU.  The
 * sender's tensor may be any view (NCCL point-to-point tolerates non-contiguous tensors,
 * torch-sys-cuda/src/nccl.rs:300-316): it is gathered in Slice::iter order into `staging`
 * (len * elem_size bytes, what an RdmaBuffer moves), and those bytes are transferred into `result`,
 * the receiver's fresh contiguous tensor of factory.size (stream.rs:1533-1538).  staging == NULL is
 * the local case from_rank == to_rank (stream.rs:1497-1516): a defensive copy straight into result.
 * result_bytes != len * elem_size -> OUTPUT_SIZE_MISMATCH. */
int mhip_send_tensor(void* result, size_t result_bytes, const void* src_base,
                     const mhip_slice_t* src_view, uint32_t elem_size, void* staging,
                     mhip_stream_t stream);

/* ====================================================================== */
/* Device-initiated RDMA: work-queue and completion-queue entries (mlx5)   */
/* ====================================================================== */
/* The NIC-free half of rdmaxcel-sys: the queue memory is whatever the caller passes (the mlx5dv_qp /
 * mlx5dv_cq buffers once they are mapped for the GPU, ordinary device or host memory otherwise); the
 * library only builds and reads the entries.  Byte layouts are rdma-core's <infiniband/mlx5dv.h>
 * (control, remote-address and data segments of 16 bytes each, big-endian fields; see
 * monarch_hip_rdmaxcel_device.h, which holds the same functions for callers' own kernels).
 * Registering queue memory for the GPU (register_cuda_memory, rdmaxcel-sys/src/rdmaxcel.c:147-207)
 * and creating queue pairs are not part of this library. */

/* wqe_params_t, rdmaxcel-sys/src/rdmaxcel.h:26-39: same fields, order and widths, hence the same
 * 80-byte layout (signaled is the reference's bool). */
typedef struct {
    uintptr_t laddr;
    uint32_t lkey;
    size_t length;
    uint64_t wr_id;
    uint8_t signaled;
    uint32_t op_type; /* MLX5_OPCODE_* */
    uintptr_t raddr;
    uint32_t rkey;
    uint32_t qp_num;
    uint8_t* buf;    /* send: mlx5dv_qp.sq.buf; receive: the slot itself */
    uint32_t* dbrec; /* mlx5dv_qp.dbrec: [0] receive, [1] send */
    uint32_t wqe_cnt;
} mhip_wqe_params_t;
/* cqe_poll_params_t, rdmaxcel.h:42-48 (32 bytes). */
typedef struct {
    uint8_t* cqe_buf;
    uint32_t cqe_size;
    uint32_t consumer_index;
    uint32_t cqe_cnt;
    uint32_t* dbrec;
} mhip_cqe_poll_params_t;
/* MLX5_OPCODE_* values RdmaQueuePair::send_wqe maps RdmaOperation to
 * (monarch_rdma/src/rdma_components.rs:1119-1124). */
enum { MHIP_MLX5_OPCODE_RDMA_WRITE = 0x08, MHIP_MLX5_OPCODE_RDMA_WRITE_IMM = 0x09, MHIP_MLX5_OPCODE_RDMA_READ = 0x10 };

/* launch_send_wqe (rdmaxcel.h:93, rdmaxcel.cu:269-275; caller monarch_rdma/src/test_utils.rs:131-160):
 * send_wqe (rdmaxcel.cu:201-245) as a kernel on `stream`.  Writes the 48 bytes of control, remote-address
 * and data segment into slot (uint32)wr_id & (wqe_cnt - 1) of buf (64-byte slots; bytes 48-63 untouched)
 * and then dbrec[1] = big-endian ((uint32)wr_id + 1) & 0xFFFFFF.  length is cut to 32 bits as in the
 * reference.  Unlike the reference's launcher it does not synchronise the device.
 * Refused with INVALID_ARGUMENT: NULL params / buf / dbrec, buf not 16-byte aligned, dbrec not 4-byte
 * aligned, wqe_cnt zero or not a power of two. */
int mhip_rdmaxcel_send_wqe(const mhip_wqe_params_t* params, mhip_stream_t stream);
/* launch_recv_wqe (rdmaxcel.h:94, rdmaxcel.cu:184-190; caller test_utils.rs:162-189): recv_wqe
 * (rdmaxcel.cu:139-160) as a kernel: one data segment at buf itself, then dbrec[0] = big-endian
 * (uint32)(wr_id + 1).  wqe_cnt is not used. */
int mhip_rdmaxcel_recv_wqe(const mhip_wqe_params_t* params, mhip_stream_t stream);
/* launch_db_ring (rdmaxcel.h:78, rdmaxcel.cu:122-124; caller test_utils.rs:191-209): db_ring
 * (rdmaxcel.cu:82-93) as a kernel: 64 bytes from src to dst as eight 64-bit stores in address order.
 * Both 8-byte aligned. */
int mhip_rdmaxcel_db_ring(void* dst, const void* src, mhip_stream_t stream);
/* RdmaQueuePair::ring_doorbell's loop (rdma_components.rs:868-885; test_utils.rs:191-209) in one launch: for
 * k = first_db_idx .. first_db_idx + count - 1 in order, db_ring(dst, sq_buf + (k % wqe_cnt) * stride), with a
 * system-scope fence between rings.  count > wqe_cnt -> MHIP_ERR_WQE_OVERFLOW ("Overflow of WQE, possible data
 * loss", rdma_components.rs:874-876).  stride is mlx5dv_qp.sq.stride, a multiple of 8 and at least 64. */
int mhip_rdmaxcel_ring_doorbells(void* dst, const void* sq_buf, uint32_t stride, uint32_t wqe_cnt,
                                 uint32_t first_db_idx, uint32_t count, mhip_stream_t stream);
/* launch_cqe_poll (rdmaxcel.h:82-84, rdmaxcel.cu:358-395; caller test_utils.rs:211-257): cqe_poll
 * (rdmaxcel.cu:292-326) as a kernel, ONE look at entry consumer_index & (cqe_cnt - 1), no spin.  The result
 * goes to the caller's device word d_result instead of a managed allocation made and freed per poll:
 * the byte count (big-endian word at byte 44 of the entry) when software owns the entry and its opcode is
 * below 4, -2 when it owns it with any other opcode, untouched otherwise; the two owned cases also store
 * big-endian (consumer_index + 1) & 0xFFFFFF at dbrec[0].  The caller sets *d_result to -1 before the call
 * (rdmaxcel.cu:293,368) and reads it after the stream has reached the kernel's end: CQE_POLL_TRUE is
 * *d_result >= 0 (rdmaxcel.cu:392).  Refused with INVALID_ARGUMENT: NULL pointers, cqe_size other than 64 or
 * 128, cqe_cnt zero or not a power of two, cqe_buf / dbrec / d_result not 4-byte aligned. */
int mhip_rdmaxcel_cqe_poll(int32_t* d_result, const mhip_cqe_poll_params_t* params, mhip_stream_t stream);

/* A transfer of params->length bytes as a chain of send WQEs in one launch: WQE i (i = 0 .. n-1, n =
 * ceil(length / max_segment_bytes)) is what send_wqe writes for {laddr + i*seg, raddr + i*seg,
 * length_i = min(seg, rest), wr_id + i} with the other fields unchanged, and the doorbell record ends at
 * ((uint32)wr_id + n) & 0xFFFFFF: the bytes n calls of mhip_rdmaxcel_send_wqe leave.  The reference posts
 * one work request per call and cuts its length to 32 bits (rdma_components.rs:1041,1063, rdmaxcel.cu:229),
 * so it has no counterpart for this; it is mhip_buffer_transfer's request walk for the device-initiated
 * path.  max_segment_bytes == 0, or anything above it, means 2^31 - 16 (bit 31 of a data segment's byte
 * count marks inline data in the mlx5 format).  *n_wqes (may be NULL) receives n.  n > wqe_cnt ->
 * MHIP_ERR_WQE_OVERFLOW; length == 0 posts one zero-length WQE, as send_wqe would. */
int mhip_rdmaxcel_post_transfer(const mhip_wqe_params_t* params, size_t max_segment_bytes,
                                uint32_t* n_wqes, mhip_stream_t stream);

/* The same functions on the calling thread, for queue memory the host can address: the reference's
 * functions are __host__ __device__ and RdmaQueuePair calls them from Rust directly
 * (send_wqe / recv_wqe: rdma_components.rs:1159-1163; db_ring: :88,:880).  Same bytes, same argument checks. */
int mhip_rdmaxcel_send_wqe_host(const mhip_wqe_params_t* params);
int mhip_rdmaxcel_recv_wqe_host(const mhip_wqe_params_t* params);
int mhip_rdmaxcel_db_ring_host(void* dst, const void* src);
int mhip_rdmaxcel_cqe_poll_host(int32_t* result, const mhip_cqe_poll_params_t* params);

/* ====================================================================== */
/* Block-scaled fp8 (e4m3fn) transfer codec                                 */
/* ====================================================================== */
/* No counterpart in the reference (fp8 tensors travel as bytes and are refused by
 * reductions, torch-sys-cuda/src/nccl.rs:275-278,474-476).  Per `block` consecutive
 * elements of a flat bf16 buffer (last block may be short):
 *   absmax = max|x| (NaN ignored) clamped to [2^-40, FLT_MAX];  scales[b] = absmax / 448
 *   q[i] = e4m3fn_rne(clamp(x[i] * (448 / absmax), -448, 448)), NaN -> the fp8 NaN code with x[i]'s sign
 * block must be 1024 (MHIP_ERR_UNSUPPORTED_BLOCK otherwise). */
int mhip_fp8_quantize(uint8_t* q, float* scales, const void* x_bf16, uint64_t numel,
                      uint32_t block, mhip_stream_t stream);
/* acc[i] += float(q[i]) * scales[i / block]; product rounded to fp32, then added. */
int mhip_fp8_dequant_accumulate(float* acc, const uint8_t* q, const float* scales, uint64_t numel,
                                uint32_t block, mhip_stream_t stream);

/* The receive side of an fp8 exchange with n peers in one pass:
 *   acc[i] = (overwrite ? 0 : acc[i]) + q[0][i]*scales[0][b] + q[1][i]*scales[1][b] + ...   (b = i / block)
 * peers in order, each product rounded before its add: bit-identical to n calls of
 * mhip_fp8_dequant_accumulate (on a zeroed accumulator when overwrite != 0), with the fp32
 * accumulator crossing HBM once.  q and scales are host tables of n device pointers, n <= 64. */
int mhip_fp8_dequant_accumulate_many(float* acc, const uint8_t* const* q, const float* const* scales,
                                     uint32_t n, uint64_t numel, uint32_t block, int overwrite,
                                     mhip_stream_t stream);

/* Fused forms on a tensor bucket (device tables as for mhip_flat_pack): bit-identical to
 * mhip_flat_pack (bf16) + mhip_fp8_quantize, resp. to mhip_fp8_dequant_accumulate on a flat
 * fp32 accumulator + mhip_flat_unpack, without materialising the flat buffers.  Blocks are
 * still counted over the bucket's flat index space.  d_tensors: bf16 inputs;
 * d_acc_tensors: fp32 accumulators, updated in place.
 * d_index is the bucket's block index (mhip_bucket_index_build) or NULL.  Without it every wavefront
 * searches the offsets table for the tensors of its span; with it that is one load.  Results are the
 * same bits either way. */
int mhip_fp8_quantize_bucket(uint8_t* q, float* scales, const void* const* d_tensors,
                             const uint64_t* d_offsets, uint32_t ntensors, uint64_t total,
                             uint32_t block, const uint32_t* d_index, mhip_stream_t stream);
int mhip_fp8_dequant_accumulate_bucket(void* const* d_acc_tensors, const uint8_t* q,
                                       const float* scales, const uint64_t* d_offsets,
                                       uint32_t ntensors, uint64_t total, uint32_t block,
                                       const uint32_t* d_index, mhip_stream_t stream);

/* mhip_fp8_dequant_accumulate_bucket for n peers in one pass (q and scales: host tables of n device
 * pointers, n <= 64): bit-identical to n single-peer calls in peer order, the accumulators cross
 * HBM once. */
int mhip_fp8_dequant_accumulate_bucket_many(void* const* d_acc_tensors, const uint8_t* const* q,
                                            const float* const* scales, uint32_t n,
                                            const uint64_t* d_offsets, uint32_t ntensors, uint64_t total,
                                            uint32_t block, const uint32_t* d_index, mhip_stream_t stream);

/* Block index of a bucket, a workspace of the fused forms above that depends on the offsets table
 * only (build it once per bucket): d_index[b] = the tensor holding flat element b * block for
 * b < ceil(total / block), and one closing entry.  *bytes = 4 * (ceil(total / block) + 1) is the
 * device memory the caller provides.  No counterpart in the reference. */
int mhip_bucket_index_bytes(uint64_t total, uint32_t block, size_t* bytes);
int mhip_bucket_index_build(uint32_t* d_index, const uint64_t* d_offsets, uint32_t ntensors,
                            uint64_t total, uint32_t block, mhip_stream_t stream);

/* mhip_fp8_quantize_bucket with the block index kept by the library: for callers that cannot allocate the
 * d_index workspace (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  The index is built into a static device array of 2^20 entries (4 MiB on every GPU
 * the library runs on) and used by the same kernel; the call allocates nothing and gives the same bits as
 * mhip_fp8_quantize_bucket.  total > (2^20 - 1) * 1024 elements -> MHIP_ERR_SCRATCH_TOO_SMALL.  All calls on one GPU
 * share that array: calls that overlap in time on one GPU (different streams, different threads) race and must
 * be ordered by the caller. */
#define MHIP_STATIC_INDEX_MAX_ELEMENTS ((((uint64_t)1 << 20) - 1) * 1024)
int mhip_fp8_quantize_bucket_static(uint8_t* q, float* scales, const void* const* d_tensors,
                                    const uint64_t* d_offsets, uint32_t ntensors, uint64_t total,
                                    uint32_t block, mhip_stream_t stream);

/* ====================================================================== */
/* Runtime pass-through (the cuda-sys / nccl-sys symbols this path uses)   */
/* ====================================================================== */
/* cuDeviceGetCount (monarch_rdma/src/test_utils.rs), cudaSetDevice (nccl-sys/build.rs:93-148) */
int mhip_device_count(int* count);
int mhip_set_device(int device);
/* cudaDeviceSynchronize (cuda-sys users in monarch_rdma/src/test_utils.rs) */
int mhip_device_synchronize(void);
/* Stream / Event of torch-sys-cuda/src/cuda.rs:30-193; default priority only. */
int mhip_stream_create(mhip_stream_t* stream);
int mhip_stream_destroy(mhip_stream_t stream);
int mhip_stream_synchronize(mhip_stream_t stream);
int mhip_event_create(mhip_event_t* event);
int mhip_event_destroy(mhip_event_t event);
int mhip_event_record(mhip_event_t event, mhip_stream_t stream);
int mhip_event_synchronize(mhip_event_t event);
int mhip_event_elapsed_ms(float* ms, mhip_event_t start, mhip_event_t stop);
int mhip_stream_wait_event(mhip_stream_t stream, mhip_event_t event);
/* cuMemcpyHtoD_v2 / cuMemcpyDtoH_v2 and device allocation for the staging-buffer test
 * environment (monarch_rdma/src/test_utils.rs:370-444). */
int mhip_malloc(void** ptr, size_t bytes);
int mhip_free(void* ptr);
int mhip_memcpy_htod(void* dst, const void* src, size_t bytes, mhip_stream_t stream);
int mhip_memcpy_dtoh(void* dst, const void* src, size_t bytes, mhip_stream_t stream);
/* Fills `bytes` bytes with the low byte of `value` (cuMemsetD8Async semantics).  Runs as a kernel, not as a memset
 * node, so it can be recorded into a HIP graph like the data-path entry points. */
int mhip_memset(void* dst, int value, size_t bytes, mhip_stream_t stream);


/* ====================================================================== */
/* Staging-buffer lifecycle (GPU memory an RdmaBuffer can register)         */
/* ====================================================================== */
/* The VMM recipe of monarch_rdma/src/test_utils.rs:370-444 (cuMemCreate / cuMemAddressReserve /
 * cuMemMap / cuMemSetAccess with a pinned device allocation): bytes are rounded up to the
 * allocation granularity, *padded_bytes receives the mapped size.  This is the one place
 * where the library allocates, and only when asked to. */
int mhip_staging_alloc(void** ptr, size_t* padded_bytes, size_t bytes, int device);
int mhip_staging_free(void* ptr, size_t padded_bytes);
/* Distance in bytes between consecutive slots of one staging area whose slots are read side by
 * side by mhip_reduce / mhip_reduce_scatter (slot r = what peer r wrote: the per-worker chunks of
 * monarch_rdma/examples/parameter_server/parameter_server.rs:193-210).  No counterpart in the
 * reference: it is a layout rule of this part's memory system.  Streams that start a multiple of
 * 16 KiB apart collide in HBM; a pitch of (slot_bytes rounded up to 16 KiB) + 8 KiB keeps them
 * apart (bf16 reduce of 8 x 48 MiB: 74.8 us at a 48 MiB pitch, 70.6 us at 48 MiB + 8 KiB). */
int mhip_staging_slot_pitch(size_t slot_bytes, size_t* pitch_bytes);
/* RdmaDomain::register_mr's first question (monarch_rdma/src/rdma_components.rs:370-377,
 * cuPointerGetAttribute(MEMORY_TYPE)): is this address device memory? */
int mhip_pointer_is_device(const void* ptr, int* is_device);
/* register_mr's second step (rdma_components.rs:386-394, cuMemGetHandleForAddressRange with
 * DMA_BUF_FD): a dma-buf file descriptor for [ptr, ptr+bytes), to hand to ibv_reg_dmabuf_mr.
 * The caller closes the descriptor. */
int mhip_export_dmabuf(int* fd, const void* ptr, size_t bytes);

#ifdef __cplusplus
}
#endif
#endif /* MONARCH_HIP_H */
