/*
 * CPU oracle for the mesh data-movement / reduce path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is a plain-C restatement of the reference's algorithms, written to be
 * checked against, never shipped: only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may load it.  Nothing in the product library links it.
 *
 * Every function cites the reference text it follows (paths relative to the
 * reference tree).  Pinning status of each group:
 *
 *   Slice algebra (new/get/iter/location/coordinates/index/select/at/subview/view/
 *     enforce_embedding/is_contiguous)            pinned: reference unit-test vectors
 *     (ndslice/src/slice.rs:835-1124, shape.rs:398-597, python/tests/_monarch/
 *     test_ndslice.py:19-167), brute force against numpy as_strided.
 *   pack / unpack                                  pinned: torch.as_strided(...).contiguous(),
 *     round-trip and tiling invariants.
 *   reduce sum (f32, exact-integer cases)          pinned: torch-sys-cuda/src/nccl.rs:850-873,
 *     1033-1065, python/tests/test_controller.py:188-254 closed forms.
 *   reduce avg, bf16 / f16 rounding, f64, reduce-scatter (f32 and bf16, Sum and Avg)
 *                                                  pinned against explicit member-order adds in numpy / torch
 *     (library routines) with n_in != n_out and strided input views; the reference holds no bf16, f64
 *     or avg vector: PARITY UNPINNED in the reference.
 *   reduce prod / max / min                        pinned against numpy multiply / fmax / fmin chains; the NaN and
 *     signed-zero rule is NCCL's, which is outside the reference tree: PARITY UNPINNED in the reference.
 *   stack (all_gather / all_to_all)                pinned: torch-sys-cuda/src/nccl.rs:927-959, 996-1031 vectors,
 *     torch.stack / chunk.
 *   send_tensor routing and result                 pinned: closed forms on the reference's mesh shapes
 *     (python/tests/test_controller.py to_mesh cases), torch .contiguous().
 *   DeviceMesh members                             pinned: monarch_tensor_worker/src/device_mesh.rs:184-244.
 *   fp8 e4m3fn block-scaled codec                  no counterpart in the reference (fp8 reductions are
 *     refused, torch-sys-cuda/src/nccl.rs:474-476): PARITY UNPINNED in the reference; the encode/decode
 *     tables are pinned against the OCP format via torch's CPU cast over all 65536 bf16 patterns.
 *   work-queue / completion-queue entries (send_wqe, recv_wqe, cqe_poll, db_ring; rdmaxcel-sys/src/rdmaxcel.cu)
 *                                                  the reference holds no byte vector (its tests need two NICs):
 *     PARITY UNPINNED in the reference; pinned by bytes written out by hand from rdma-core's published mlx5 segment
 *     layouts (tests/test_oracle_rdmaxcel.py), sixteen source mutations of these functions each fail one of them.
 */
#ifdef _OPENMP
#include <omp.h>
#endif
#include <math.h>
#include <float.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- error classes: one per SliceError variant, ndslice/src/slice.rs:15-51 ---- */
enum {
    O_OK = 0,
    O_ERR_INVALID_DIMS = 1,
    O_ERR_NONRECTANGULAR = 2,
    O_ERR_NONUNIQUE_STRIDES = 3,
    O_ERR_STRIDE_TOO_SMALL = 4,
    O_ERR_INDEX_OUT_OF_RANGE = 5,
    O_ERR_VALUE_NOT_IN_SLICE = 6,
    O_ERR_INCOMPATIBLE_VIEW = 7,
    O_ERR_NONCONTIGUOUS = 8,
    O_ERR_EMPTY_RANGE = 9,
    O_ERR_DIM_OUT_OF_RANGE = 10,
};

typedef struct {
    uint64_t offset;
    uint32_t ndim;
    const uint64_t* sizes;
    const uint64_t* strides;
} o_slice_t;

/* Slice::new validation, ndslice/src/slice.rs:99-139.  `nstrides` is passed
 * separately so the InvalidDims branch (:100-105) can be exercised. */
int o_slice_new(uint64_t offset, const uint64_t* sizes, uint32_t nsizes, const uint64_t* strides,
                uint32_t nstrides) {
    (void)offset;
    if (nsizes != nstrides) return O_ERR_INVALID_DIMS;
    uint32_t n = nsizes;
    uint64_t* st = (uint64_t*)malloc(sizeof(uint64_t) * (n ? n : 1));
    uint64_t* sz = (uint64_t*)malloc(sizeof(uint64_t) * (n ? n : 1));
    /* combined.sort(): lexicographic on (stride, size), :106-108 */
    for (uint32_t i = 0; i < n; i++) {
        uint64_t s = strides[i], z = sizes[i];
        uint32_t j = i;
        while (j > 0 && (st[j - 1] > s || (st[j - 1] == s && sz[j - 1] > z))) {
            st[j] = st[j - 1];
            sz[j] = sz[j - 1];
            j--;
        }
        st[j] = s;
        sz[j] = z;
    }
    int rc = O_OK;
    int have_prev = 0;
    uint64_t prev_stride = 0, prev_size = 1, total = 1;
    for (uint32_t i = 0; i < n; i++) {
        uint64_t stride = st[i], size = sz[i];
        if (have_prev) {
            if (stride % prev_stride != 0) { rc = O_ERR_NONRECTANGULAR; break; }      /* :115-117 */
            if (stride == prev_stride && size != 1 && prev_size != 1) {                /* :119-121 */
                rc = O_ERR_NONUNIQUE_STRIDES;
                break;
            }
        }
        if (total > stride) { rc = O_ERR_STRIDE_TOO_SMALL; break; }                    /* :123-128 */
        total = stride * size;
        prev_stride = stride;
        prev_size = size;
        have_prev = 1;
    }
    free(st);
    free(sz);
    return rc;
}

/* Slice::len, slice.rs:382-384 (empty product = 1). */
uint64_t o_slice_len(const o_slice_t* s) {
    uint64_t n = 1;
    for (uint32_t i = 0; i < s->ndim; i++) n *= s->sizes[i];
    return n;
}

/* Slice::is_contiguous, slice.rs:198-207. */
int o_slice_is_contiguous(const o_slice_t* s) {
    uint64_t expected = 1;
    for (uint32_t k = s->ndim; k-- > 0;) {
        if (s->strides[k] != expected) return 0;
        expected *= s->sizes[k];
    }
    return 1;
}

/* Slice::location, slice.rs:330-343. */
int o_slice_location(const o_slice_t* s, const uint64_t* coord, uint32_t ncoord, uint64_t* out) {
    if (ncoord != s->ndim) return O_ERR_INVALID_DIMS;
    uint64_t v = s->offset;
    for (uint32_t k = 0; k < s->ndim; k++) v += coord[k] * s->strides[k];
    *out = v;
    return O_OK;
}

/* Slice::get, slice.rs:523-537.  A zero size makes the reference divide by zero
 * (:529); the oracle reports IndexOutOfRange instead, since len()==0 there. */
int o_slice_get(const o_slice_t* s, uint64_t index, uint64_t* out) {
    uint64_t val = s->offset, rest = index, total = 1;
    for (uint32_t k = s->ndim; k-- > 0;) {
        uint64_t size = s->sizes[k];
        if (size == 0) return O_ERR_INDEX_OUT_OF_RANGE;
        total *= size;
        val += (rest % size) * s->strides[k];
        rest /= size;
    }
    if (index < total) {
        *out = val;
        return O_OK;
    }
    return O_ERR_INDEX_OUT_OF_RANGE;
}

/* CartesianIterator::next, slice.rs:764-781, followed by SliceIterator::next,
 * :709-718: the i-th item is location(coords(i)).  Writes min(len, cap) items and
 * returns len. */
uint64_t o_slice_iter(const o_slice_t* s, uint64_t* out, uint64_t cap) {
    uint64_t len = o_slice_len(s);
    uint64_t coord[64];
    for (uint64_t index = 0; index < len && index < cap; index++) {
        uint64_t rest = index;
        for (uint32_t k = s->ndim; k-- > 0;) {
            coord[k] = rest % s->sizes[k];
            rest /= s->sizes[k];
        }
        uint64_t loc;
        o_slice_location(s, coord, s->ndim, &loc);
        out[index] = loc;
    }
    return len;
}

/* Slice::coordinates, slice.rs:347-374: peel by descending stride, size-1 dims
 * take coordinate 0 and do not consume position.  sort_by_key is stable. */
int o_slice_coordinates(const o_slice_t* s, uint64_t value, uint64_t* out) {
    if (value < s->offset) return O_ERR_VALUE_NOT_IN_SLICE;
    uint64_t pos = value - s->offset;
    uint32_t n = s->ndim;
    uint32_t order[64];
    for (uint32_t i = 0; i < n; i++) {
        uint32_t j = i;
        while (j > 0 && s->strides[order[j - 1]] > s->strides[i]) {
            order[j] = order[j - 1];
            j--;
        }
        order[j] = i;
    }
    for (uint32_t i = 0; i < n; i++) out[i] = 0;
    for (uint32_t r = n; r-- > 0;) {
        uint32_t i = order[r];
        uint64_t stride = s->strides[i], size = s->sizes[i];
        uint64_t index, new_pos;
        if (size > 1) {
            index = pos / stride;
            new_pos = pos % stride;
        } else {
            index = 0;
            new_pos = pos;
        }
        if (index >= size) return O_ERR_VALUE_NOT_IN_SLICE;
        out[i] = index;
        pos = new_pos;
    }
    if (pos != 0) return O_ERR_VALUE_NOT_IN_SLICE;
    return O_OK;
}

/* Slice::index, slice.rs:460-471. */
int o_slice_index(const o_slice_t* s, uint64_t value, uint64_t* out) {
    uint64_t coords[64];
    int rc = o_slice_coordinates(s, value, coords);
    if (rc) return rc;
    uint64_t stride = 1, result = 0;
    for (uint32_t k = s->ndim; k-- > 0;) {
        result += coords[k] * stride;
        stride *= s->sizes[k];
    }
    *out = result;
    return O_OK;
}

/* Slice::select, slice.rs:291-327.  Outputs have ndim entries. */
int o_slice_select(const o_slice_t* s, uint32_t dim, uint64_t begin, uint64_t end, uint64_t step,
                   uint64_t* out_offset, uint64_t* out_sizes, uint64_t* out_strides) {
    if (dim >= s->ndim) return O_ERR_INDEX_OUT_OF_RANGE;
    if (begin >= s->sizes[dim]) return O_ERR_INDEX_OUT_OF_RANGE;
    if (end <= begin) return O_ERR_EMPTY_RANGE;
    uint64_t offset = s->offset;
    for (uint32_t k = 0; k < s->ndim; k++) {
        out_sizes[k] = s->sizes[k];
        out_strides[k] = s->strides[k];
    }
    offset += begin * out_strides[dim];
    out_sizes[dim] = (end - begin + step - 1) / step; /* div_ceil, :322 */
    out_strides[dim] *= step;
    *out_offset = offset;
    return o_slice_new(offset, out_sizes, s->ndim, out_strides, s->ndim); /* :325 */
}

/* Slice::at, slice.rs:243-264.  Outputs have ndim-1 entries. */
int o_slice_at(const o_slice_t* s, uint32_t dim, uint64_t index, uint64_t* out_offset,
               uint64_t* out_sizes, uint64_t* out_strides) {
    if (dim >= s->ndim) return O_ERR_DIM_OUT_OF_RANGE;
    if (index >= s->sizes[dim]) return O_ERR_INDEX_OUT_OF_RANGE;
    *out_offset = s->offset + index * s->strides[dim];
    uint32_t j = 0;
    for (uint32_t k = 0; k < s->ndim; k++) {
        if (k == dim) continue;
        out_sizes[j] = s->sizes[k];
        out_strides[j] = s->strides[k];
        j++;
    }
    return o_slice_new(*out_offset, out_sizes, s->ndim - 1, out_strides, s->ndim - 1); /* :262 */
}

/* Slice::subview, slice.rs:638-661 (no re-validation). */
int o_slice_subview(const o_slice_t* s, const uint64_t* starts, uint32_t nstarts,
                    const uint64_t* lens, uint32_t nlens, uint64_t* out_offset) {
    if (nstarts != s->ndim || nlens != s->ndim) return O_ERR_INVALID_DIMS;
    for (uint32_t d = 0; d < s->ndim; d++)
        if (starts[d] + lens[d] > s->sizes[d]) return O_ERR_INDEX_OUT_OF_RANGE;
    return o_slice_location(s, starts, nstarts, out_offset);
}

/* Slice::view, slice.rs:579-635.  out_strides has nnew entries. */
int o_slice_view(const o_slice_t* s, const uint64_t* new_sizes, uint32_t nnew,
                 uint64_t* out_strides) {
    uint64_t view_elems = 1, base_elems = o_slice_len(s);
    for (uint32_t i = 0; i < nnew; i++) view_elems *= new_sizes[i];
    if (view_elems != base_elems) return O_ERR_INCOMPATIBLE_VIEW;
    if (s->offset != 0) return O_ERR_INCOMPATIBLE_VIEW;
    for (uint32_t i = 0; i < nnew; i++) out_strides[i] = 1;
    if (nnew >= 2)
        for (uint32_t i = nnew - 1; i-- > 0;) out_strides[i] = out_strides[i + 1] * new_sizes[i + 1];
    uint64_t coords[64], tmp[64];
    for (uint64_t idx = 0; idx < view_elems; idx++) {
        uint64_t rest = idx, off = 0;
        for (uint32_t k = nnew; k-- > 0;) {
            coords[k] = rest % new_sizes[k];
            rest /= new_sizes[k];
        }
        for (uint32_t k = 0; k < nnew; k++) off += coords[k] * out_strides[k];
        if (o_slice_coordinates(s, off, tmp) != O_OK) return O_ERR_INCOMPATIBLE_VIEW;
    }
    return O_OK;
}

/* Slice::enforce_embedding, slice.rs:683-687. */
int o_slice_enforce_embedding(const o_slice_t* s, const o_slice_t* other) {
    uint64_t len = o_slice_len(s), tmp[64];
    for (uint64_t i = 0; i < len; i++) {
        uint64_t loc;
        int rc = o_slice_get(s, i, &loc);
        if (rc) return rc;
        rc = o_slice_coordinates(other, loc, tmp);
        if (rc) return rc;
    }
    return O_OK;
}

/* ---- pack / unpack: the staging copy defined by Slice::iter order ----
 * dst[i] = src[get(i)] (pack) and dst[get(i)] = src[i] (unpack), i in [0, len),
 * elementwise over `elem_size`-byte elements.  This is the literal per-element
 * div/mod walk of slice.rs:523-537 and :764-781. */
void o_slice_pack(void* dst, const void* src_base, const o_slice_t* s, uint32_t elem_size) {
    uint64_t len = o_slice_len(s);
    for (uint64_t i = 0; i < len; i++) {
        uint64_t loc;
        o_slice_get(s, i, &loc);
        memcpy((char*)dst + i * elem_size, (const char*)src_base + loc * elem_size, elem_size);
    }
}

void o_slice_unpack(void* dst_base, const void* src, const o_slice_t* s, uint32_t elem_size) {
    uint64_t len = o_slice_len(s);
    for (uint64_t i = 0; i < len; i++) {
        uint64_t loc;
        o_slice_get(s, i, &loc);
        memcpy((char*)dst_base + loc * elem_size, (const char*)src + i * elem_size, elem_size);
    }
}

/* ---- bf16 helpers: round-to-nearest-even on the top 16 bits of an fp32 ---- */
static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint16_t f32_to_bf16_rne(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0; /* NaN -> canonical quiet NaN */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}
void o_bf16_to_f32(float* out, const uint16_t* in, uint64_t n) {
    for (uint64_t i = 0; i < n; i++) out[i] = bf16_to_f32(in[i]);
}
void o_f32_to_bf16(uint16_t* out, const float* in, uint64_t n) {
    for (uint64_t i = 0; i < n; i++) out[i] = f32_to_bf16_rne(in[i]);
}

/* ---- IEEE binary16 helpers (widening exact, narrowing round-to-nearest-even) ---- */
static inline float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1f, m = h & 0x3ffu;
    float v;
    if (e == 0)
        v = ldexpf((float)m, -24); /* zero and subnormals */
    else if (e == 31) {
        uint32_t u = 0x7f800000u | (m << 13);
        memcpy(&v, &u, 4);
    } else
        v = ldexpf((float)(m | 0x400u), (int)e - 25);
    uint32_t u;
    memcpy(&u, &v, 4);
    u |= sign;
    memcpy(&v, &u, 4);
    return v;
}
static inline uint16_t f32_to_f16_rne(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u); /* NaN -> quiet NaN */
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536: infinity (also catches inf) */
    float av;
    memcpy(&av, &a, 4);
    if (a < 0x38800000u) { /* below 2^-14: subnormal grid of 2^-24 */
        uint32_t m = (uint32_t)rintf(ldexpf(av, 24));
        return (uint16_t)(sign | m); /* m == 1024 lands on the smallest normal */
    }
    int ex;
    float fr = frexpf(av, &ex); /* av = fr * 2^ex, fr in [0.5, 1) */
    uint32_t m = (uint32_t)rintf((2.0f * fr - 1.0f) * 1024.0f);
    int e = ex - 1 + 15;
    if (m == 1024) {
        m = 0;
        e += 1;
    }
    if (e >= 31) return (uint16_t)(sign | 0x7c00u); /* 65520 and above round to infinity */
    return (uint16_t)(sign | ((uint32_t)e << 10) | m);
}
void o_f16_to_f32(float* out, const uint16_t* in, uint64_t n) {
    for (uint64_t i = 0; i < n; i++) out[i] = f16_to_f32(in[i]);
}
void o_f32_to_f16(uint16_t* out, const float* in, uint64_t n) {
    for (uint64_t i = 0; i < n; i++) out[i] = f32_to_f16_rne(in[i]);
}

/* ---- Reduce, non-scatter: out = op over the n chunks this GPU holds ----
 * Semantics of StreamActor::reduce's all_reduce branch
 * (monarch_tensor_worker/src/stream.rs:1437-1462; python/monarch/worker/worker.py:251-255):
 * elementwise over n same-shaped inputs.  Accumulation is fp32, left to right in
 * rank order, Avg divides the fp32 sum by n, bf16 results are rounded once at the
 * end.  The loop shape is that of the reference's own CPU accumulate
 * (monarch_rdma/examples/parameter_server/parameter_server.rs:200-205).
 * `out` may alias in[0].  op: 0 = Sum, 4 = Avg (torch-sys-cuda/src/nccl.rs:285-292). */
void o_reduce_f32(float* out, const float* const* in, uint32_t n, uint64_t numel, int op) {
    for (uint64_t i = 0; i < numel; i++) {
        float acc = in[0][i];
        for (uint32_t r = 1; r < n; r++) acc += in[r][i];
        if (op == 4) acc = acc / (float)n;
        out[i] = acc;
    }
}
void o_reduce_bf16(uint16_t* out, const uint16_t* const* in, uint32_t n, uint64_t numel, int op) {
    for (uint64_t i = 0; i < numel; i++) {
        float acc = bf16_to_f32(in[0][i]);
        for (uint32_t r = 1; r < n; r++) acc += bf16_to_f32(in[r][i]);
        if (op == 4) acc = acc / (float)n;
        out[i] = f32_to_bf16_rne(acc);
    }
}
void o_reduce_f16(uint16_t* out, const uint16_t* const* in, uint32_t n, uint64_t numel, int op) {
    for (uint64_t i = 0; i < numel; i++) {
        float acc = f16_to_f32(in[0][i]);
        for (uint32_t r = 1; r < n; r++) acc += f16_to_f32(in[r][i]);
        if (op == 4) acc = acc / (float)n;
        out[i] = f32_to_f16_rne(acc);
    }
}
void o_reduce_f64(double* out, const double* const* in, uint32_t n, uint64_t numel, int op) {
    for (uint64_t i = 0; i < numel; i++) {
        double acc = in[0][i];
        for (uint32_t r = 1; r < n; r++) acc += in[r][i];
        if (op == 4) acc = acc / (double)n;
        out[i] = acc;
    }
}
/* Integer Sum wraps, as the parameter server's u8 wrapping_add does
 * (parameter_server.rs:202). */
void o_reduce_u8(uint8_t* out, const uint8_t* const* in, uint32_t n, uint64_t numel) {
    for (uint64_t i = 0; i < numel; i++) {
        uint8_t acc = in[0][i];
        for (uint32_t r = 1; r < n; r++) acc = (uint8_t)(acc + in[r][i]);
        out[i] = acc;
    }
}
void o_reduce_i32(int32_t* out, const int32_t* const* in, uint32_t n, uint64_t numel) {
    for (uint64_t i = 0; i < numel; i++) {
        uint32_t acc = (uint32_t)in[0][i];
        for (uint32_t r = 1; r < n; r++) acc += (uint32_t)in[r][i];
        out[i] = (int32_t)acc;
    }
}
void o_reduce_i64(int64_t* out, const int64_t* const* in, uint32_t n, uint64_t numel) {
    for (uint64_t i = 0; i < numel; i++) {
        uint64_t acc = (uint64_t)in[0][i];
        for (uint32_t r = 1; r < n; r++) acc += (uint64_t)in[r][i];
        out[i] = (int64_t)acc;
    }
}

static float o_combine_f32(float acc, float x, int op); /* defined with the other ops below */

/* ---- Reduce with scatter ----
 * reduced[i] = op_g in[g][in_view.get(i)] over the logical index space of in_view;
 * outs[k][j] = reduced[out_views[k].get(j)].  With in_view contiguous [n*c] and
 * out_views[k] = {k*c,[c],[1]} this is ncclReduceScatter's flat-chunk rule
 * (torch-sys-cuda/src/nccl.rs:683,693-701; stream.rs:1422-1436). */
void o_reduce_scatter_f32(float* const* outs, const o_slice_t* out_views, uint32_t n_out,
                          const float* const* in, const o_slice_t* in_view, uint32_t n_in, int op) {
    for (uint32_t k = 0; k < n_out; k++) {
        uint64_t len = o_slice_len(&out_views[k]);
        for (uint64_t j = 0; j < len; j++) {
            uint64_t i, loc;
            o_slice_get(&out_views[k], j, &i);
            o_slice_get(in_view, i, &loc);
            float acc = in[0][loc];
            for (uint32_t g = 1; g < n_in; g++) acc = o_combine_f32(acc, in[g][loc], op);
            if (op == 4) acc = acc / (float)n_in;
            outs[k][j] = acc;
        }
    }
}
void o_reduce_scatter_bf16(uint16_t* const* outs, const o_slice_t* out_views, uint32_t n_out,
                           const uint16_t* const* in, const o_slice_t* in_view, uint32_t n_in,
                           int op) {
    for (uint32_t k = 0; k < n_out; k++) {
        uint64_t len = o_slice_len(&out_views[k]);
        for (uint64_t j = 0; j < len; j++) {
            uint64_t i, loc;
            o_slice_get(&out_views[k], j, &i);
            o_slice_get(in_view, i, &loc);
            float acc = bf16_to_f32(in[0][loc]);
            for (uint32_t g = 1; g < n_in; g++) acc = o_combine_f32(acc, bf16_to_f32(in[g][loc]), op);
            if (op == 4) acc = acc / (float)n_in;
            outs[k][j] = f32_to_bf16_rne(acc);
        }
    }
}

/* ---- The other ReduceOps (torch-sys-cuda/src/nccl.rs:285-292: Prod = 1, Max = 2, Min = 3) ----
 * Same shape as the Sum loops above: accumulate in member order in fp32 (f64 for f64, the integer
 * type for integers), round once.  Max / Min are written out as comparisons so that every case is
 * fixed: the accumulator is kept on ties (the first of +0 / -0 in member order wins) and a NaN operand
 * is skipped unless all operands are NaN - the result fmaxf / fminf give, which is how NCCL's kernels
 * compute ncclMax / ncclMin.  NCCL itself is not part of the reference tree and the reference holds no
 * vector for these ops: PARITY UNPINNED against the reference; pinned against numpy (fmax / fmin /
 * multiply) only.  Integer Prod wraps, as integer Sum does (parameter_server.rs:202). */
static float o_combine_f32(float acc, float x, int op) {
    switch (op) {
        case 1: return acc * x;
        case 2: return (x > acc || acc != acc) ? x : acc;
        case 3: return (x < acc || acc != acc) ? x : acc;
        default: return acc + x;
    }
}
static double o_combine_f64(double acc, double x, int op) {
    switch (op) {
        case 1: return acc * x;
        case 2: return (x > acc || acc != acc) ? x : acc;
        case 3: return (x < acc || acc != acc) ? x : acc;
        default: return acc + x;
    }
}
#define O_INT_COMBINE(NAME, T, UT)                                 \
    static T NAME(T acc, T x, int op) {                            \
        switch (op) {                                              \
            case 1: return (T)(UT)((UT)acc * (UT)x);               \
            case 2: return x > acc ? x : acc;                      \
            case 3: return x < acc ? x : acc;                      \
            default: return (T)(UT)((UT)acc + (UT)x);              \
        }                                                          \
    }
O_INT_COMBINE(o_combine_u8, uint8_t, uint8_t)
O_INT_COMBINE(o_combine_i8, int8_t, uint8_t)
O_INT_COMBINE(o_combine_i32, int32_t, uint32_t)
O_INT_COMBINE(o_combine_i64, int64_t, uint64_t)

/* out = op over the n inputs for any ReduceOp; dtype in c10::ScalarType numbering
 * (0 u8, 1 i8, 3 i32, 4 i64, 5 f16, 6 f32, 7 f64, 15 bf16).  Returns 0, or -1 for an unknown dtype. */
int o_reduce_op(void* out, const void* const* in, uint32_t n, uint64_t numel, int dtype, int op) {
    for (uint64_t i = 0; i < numel; i++) {
        switch (dtype) {
            case 6: {
                float acc = ((const float*)in[0])[i];
                for (uint32_t r = 1; r < n; r++) acc = o_combine_f32(acc, ((const float*)in[r])[i], op);
                if (op == 4) acc = acc / (float)n;
                ((float*)out)[i] = acc;
                break;
            }
            case 15: {
                float acc = bf16_to_f32(((const uint16_t*)in[0])[i]);
                for (uint32_t r = 1; r < n; r++) acc = o_combine_f32(acc, bf16_to_f32(((const uint16_t*)in[r])[i]), op);
                if (op == 4) acc = acc / (float)n;
                ((uint16_t*)out)[i] = f32_to_bf16_rne(acc);
                break;
            }
            case 5: {
                float acc = f16_to_f32(((const uint16_t*)in[0])[i]);
                for (uint32_t r = 1; r < n; r++) acc = o_combine_f32(acc, f16_to_f32(((const uint16_t*)in[r])[i]), op);
                if (op == 4) acc = acc / (float)n;
                ((uint16_t*)out)[i] = f32_to_f16_rne(acc);
                break;
            }
            case 7: {
                double acc = ((const double*)in[0])[i];
                for (uint32_t r = 1; r < n; r++) acc = o_combine_f64(acc, ((const double*)in[r])[i], op);
                if (op == 4) acc = acc / (double)n;
                ((double*)out)[i] = acc;
                break;
            }
            case 0: {
                uint8_t acc = ((const uint8_t*)in[0])[i];
                for (uint32_t r = 1; r < n; r++) acc = o_combine_u8(acc, ((const uint8_t*)in[r])[i], op);
                ((uint8_t*)out)[i] = acc;
                break;
            }
            case 1: {
                int8_t acc = ((const int8_t*)in[0])[i];
                for (uint32_t r = 1; r < n; r++) acc = o_combine_i8(acc, ((const int8_t*)in[r])[i], op);
                ((int8_t*)out)[i] = acc;
                break;
            }
            case 3: {
                int32_t acc = ((const int32_t*)in[0])[i];
                for (uint32_t r = 1; r < n; r++) acc = o_combine_i32(acc, ((const int32_t*)in[r])[i], op);
                ((int32_t*)out)[i] = acc;
                break;
            }
            case 4: {
                int64_t acc = ((const int64_t*)in[0])[i];
                for (uint32_t r = 1; r < n; r++) acc = o_combine_i64(acc, ((const int64_t*)in[r])[i], op);
                ((int64_t*)out)[i] = acc;
                break;
            }
            default: return -1;
        }
    }
    return 0;
}

/* ---- Reduction::Stack ----
 * Without scatter: all_gather_into_tensor (monarch_tensor_worker/src/stream.rs:1408-1417), result
 * [n, *shape]: out[g*numel + i] = in[g][i]; the reference's vector is torch-sys-cuda/src/nccl.rs:927-959. */
void o_stack(void* out, const void* const* in, uint32_t n, uint64_t numel, uint32_t elem_size) {
    for (uint32_t g = 0; g < n; g++)
        for (uint64_t b = 0; b < numel * elem_size; b++)
            ((uint8_t*)out)[(uint64_t)g * numel * elem_size + b] = ((const uint8_t*)in[g])[b];
}
/* With scatter: all_to_all_single (stream.rs:1381-1399; nccl.rs:760-812: count = numel / world_size,
 * chunk r of the send buffer goes to rank r, the chunk received from rank r lands at chunk r) as
 * member `rank` sees it: out[g*c + i] = in[g][rank*c + i].  Vector: nccl.rs:996-1031.  `out` is written
 * through a temporary so that the in-place form (out == in[rank]) reads pre-exchange values. */
int o_stack_scatter(void* out, const void* const* in, uint32_t n, uint32_t rank, uint64_t numel,
                    uint32_t elem_size) {
    if (n == 0 || numel % n != 0 || rank >= n) return -1;
    uint64_t chunk = numel / n * elem_size;
    uint8_t* tmp = (uint8_t*)malloc(chunk * n + 1);
    if (!tmp) return -2;
    for (uint32_t g = 0; g < n; g++) memcpy(tmp + g * chunk, (const uint8_t*)in[g] + rank * chunk, chunk);
    memcpy(out, tmp, chunk * n);
    free(tmp);
    return 0;
}

/* ---- SendTensor ----
 * Routing, monarch_tensor_worker/src/lib.rs:722-731: to_rank = to_ranks.get(from_ranks.index(rank)),
 * from_rank = from_ranks.get(to_ranks.index(rank)); UINT64_MAX stands for None. */
void o_send_tensor_route(const o_slice_t* from_ranks, const o_slice_t* to_ranks, uint64_t rank,
                         uint64_t* from_rank, uint64_t* to_rank) {
    uint64_t index, peer;
    *to_rank = *from_rank = UINT64_MAX;
    if (o_slice_index(from_ranks, rank, &index) == O_OK && o_slice_get(to_ranks, index, &peer) == O_OK)
        *to_rank = peer;
    if (o_slice_index(to_ranks, rank, &index) == O_OK && o_slice_get(from_ranks, index, &peer) == O_OK)
        *from_rank = peer;
}
/* What StreamActor::send_tensor (stream.rs:1470-1560) leaves on the receiver: a fresh contiguous tensor
 * of factory.size holding the sender's elements in logical (row-major, Slice::iter) order.  The sender's
 * view goes through staging bytes, the transfer is a byte copy. */
void o_send_tensor(void* result, const void* src_base, const o_slice_t* src_view, uint32_t elem_size) {
    uint64_t bytes = o_slice_len(src_view) * elem_size;
    uint8_t* staging = (uint8_t*)malloc(bytes ? bytes : 1);
    o_slice_pack(staging, src_base, src_view, elem_size);
    memcpy(result, staging, bytes);
    free(staging);
}

/* ---- DeviceMesh, monarch_tensor_worker/src/device_mesh.rs:71-102 ----
 * Members of dimension `dim` for the owning `rank`:
 * start = rank - stride*coord; members = start, start+stride, ... (size items). */
int o_mesh_dim_members(const o_slice_t* ranks, uint64_t rank, uint32_t dim, uint64_t* members,
                       uint64_t* dim_rank) {
    uint64_t coords[64];
    int rc = o_slice_coordinates(ranks, rank, coords);
    if (rc) return rc;
    if (dim >= ranks->ndim) return O_ERR_DIM_OUT_OF_RANGE;
    uint64_t stride = ranks->strides[dim], size = ranks->sizes[dim];
    uint64_t start = rank - stride * coords[dim];
    for (uint64_t i = 0; i < size; i++) members[i] = start + i * stride;
    *dim_rank = coords[dim];
    return O_OK;
}

/* get_ranks_for_dim_slice, device_mesh.rs:120-177: cartesian product over the
 * named dims, in the order given.  Returns the count (0 for no dims). */
int64_t o_mesh_ranks_for_dims(const o_slice_t* ranks, uint64_t rank, const uint32_t* dims,
                              uint32_t ndims, uint64_t* out) {
    if (ndims == 0) return 0;
    uint64_t coords[64];
    if (o_slice_coordinates(ranks, rank, coords)) return -1;
    uint64_t strides[64], sizes[64], total = 1, start = rank;
    for (uint32_t d = 0; d < ndims; d++) {
        if (dims[d] >= ranks->ndim) return -1;
        sizes[d] = ranks->sizes[dims[d]];
        /* :148-154: stride is members[1]-members[0], or 0 for a 1-member dim */
        strides[d] = sizes[d] >= 2 ? ranks->strides[dims[d]] : 0;
        total *= sizes[d];
        start -= strides[d] * coords[dims[d]];
    }
    for (uint64_t idx = 0; idx < total; idx++) {
        uint64_t rest = idx, v = start;
        for (uint32_t d = ndims; d-- > 0;) {
            v += (rest % sizes[d]) * strides[d];
            rest /= sizes[d];
        }
        out[idx] = v;
    }
    return (int64_t)total;
}

/* ---- fp8 e4m3fn (OCP 8-bit float, 4 exponent bits bias 7, 3 mantissa bits,
 * no infinity, NaN = S.1111.111, max finite 448, min subnormal 2^-9) ----
 * The reference has no fp8 arithmetic (fp8 tensors travel as bytes,
 * torch-sys-cuda/src/nccl.rs:275-278, and reductions on them are refused,
 * :474-476); the format definition is the oracle. */
uint8_t o_e4m3fn_encode(float f, int saturate) {
    uint32_t u;
    memcpy(&u, &f, 4);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint8_t)(sign | 0x7f);
    float a = fabsf(f);
    if (isinf(a)) return (uint8_t)(sign | (saturate ? 0x7e : 0x7f));
    if (a < 0.015625f) { /* below 2^-6: subnormal grid of 2^-9 */
        int m = (int)rintf(ldexpf(a, 9));
        return (uint8_t)(sign | m); /* m == 8 lands on 0x08, the min normal */
    }
    int ex;
    float fr = frexpf(a, &ex); /* a = fr * 2^ex, fr in [0.5, 1) */
    int e = ex - 1;
    int m = (int)rintf((2.0f * fr - 1.0f) * 8.0f);
    if (m == 8) {
        m = 0;
        e += 1;
    }
    if (e > 8 || (e == 8 && m == 7)) return (uint8_t)(sign | (saturate ? 0x7e : 0x7f));
    return (uint8_t)(sign | ((e + 7) << 3) | m);
}

float o_e4m3fn_decode(uint8_t c) {
    int e = (c >> 3) & 0xf, m = c & 7;
    float v;
    if (e == 15 && m == 7)
        v = NAN;
    else if (e == 0)
        v = ldexpf((float)m, -9);
    else
        v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return (c & 0x80) ? -v : v;
}

/* Block-scaled quantisation of a flat bf16 buffer.  Per `block` consecutive
 * elements (the last block may be short):
 *   absmax = max |x| (NaN ignored), clamped to [2^-40, FLT_MAX]
 *   scale  = absmax / 448            (stored, fp32)
 *   inv    = 448 / absmax
 *   y      = x * inv, clamped to [-448, 448] by comparisons that let NaN through
 *   q      = e4m3fn_rne(y)
 */
#define O_FP8_MAX 448.0f
#define O_FP8_EPS 9.094947017729282e-13f /* 2^-40 */
void o_fp8_quantize(uint8_t* q, float* scales, const uint16_t* x, uint64_t numel, uint32_t block) {
    uint64_t nblocks = (numel + block - 1) / block;
    for (uint64_t b = 0; b < nblocks; b++) {
        uint64_t lo = b * block, hi = lo + block < numel ? lo + block : numel;
        float absmax = 0.0f;
        for (uint64_t i = lo; i < hi; i++) {
            float a = fabsf(bf16_to_f32(x[i]));
            if (a > absmax) absmax = a;
        }
        if (absmax < O_FP8_EPS) absmax = O_FP8_EPS;
        if (absmax > FLT_MAX) absmax = FLT_MAX;
        float scale = absmax / O_FP8_MAX;
        float inv = O_FP8_MAX / absmax;
        scales[b] = scale;
        for (uint64_t i = lo; i < hi; i++) {
            float y = bf16_to_f32(x[i]) * inv;
            if (y > O_FP8_MAX) y = O_FP8_MAX;
            if (y < -O_FP8_MAX) y = -O_FP8_MAX;
            q[i] = o_e4m3fn_encode(y, 1);
        }
    }
}

/* acc[i] += decode(q[i]) * scale[i / block]; the product is rounded to fp32
 * before the add (two roundings, no fused multiply-add). */
void o_fp8_dequant_accumulate(float* acc, const uint8_t* q, const float* scales, uint64_t numel,
                              uint32_t block) {
    for (uint64_t i = 0; i < numel; i++) {
        volatile float xhat = o_e4m3fn_decode(q[i]) * scales[i / block];
        acc[i] = acc[i] + xhat;
    }
}
void o_fp8_dequantize(float* out, const uint8_t* q, const float* scales, uint64_t numel,
                      uint32_t block) {
    for (uint64_t i = 0; i < numel; i++) out[i] = o_e4m3fn_decode(q[i]) * scales[i / block];
}

/* Flat buffer with an offsets table: the torch.cat / split pair of a gradient
 * bucket (python/tests/simulator/test_simulator.py:190-203) generalised to ragged
 * tensors.  offsets has ntensors+1 entries, in elements. */
void o_flat_pack(void* flat, const void* const* tensors, const uint64_t* offsets, uint32_t ntensors,
                 uint32_t elem_size) {
    for (uint32_t t = 0; t < ntensors; t++)
        memcpy((char*)flat + offsets[t] * elem_size, tensors[t],
               (offsets[t + 1] - offsets[t]) * elem_size);
}
void o_flat_unpack(void* const* tensors, const void* flat, const uint64_t* offsets,
                   uint32_t ntensors, uint32_t elem_size) {
    for (uint32_t t = 0; t < ntensors; t++)
        memcpy(tensors[t], (const char*)flat + offsets[t] * elem_size,
               (offsets[t + 1] - offsets[t]) * elem_size);
}

/* ---- timed CPU baselines for bench.py (single thread, same loops as above) ---- */
void o_pack_runs(void* dst, const void* src_base, const o_slice_t* s, uint32_t elem_size) {
    /* fair CPU path: memcpy per innermost contiguous run when the last stride is 1 */
    if (s->ndim == 0 || s->strides[s->ndim - 1] != 1) {
        o_slice_pack(dst, src_base, s, elem_size);
        return;
    }
    uint64_t run = s->sizes[s->ndim - 1];
    uint64_t len = o_slice_len(s);
    for (uint64_t i = 0; i < len; i += run) {
        uint64_t loc;
        o_slice_get(s, i, &loc);
        memcpy((char*)dst + i * elem_size, (const char*)src_base + loc * elem_size,
               run * elem_size);
    }
}

/* ---- the same two loops on every host core (OpenMP): the "fair" CPU figures that
 * bench.py reports beside the single-thread restatement, so that the GPU is not only
 * compared with a scalar loop.  Results are identical to the single-thread functions:
 * rows (pack) and elements (reduce) are independent. */
void o_pack_runs_mt(void* dst, const void* src_base, const o_slice_t* s, uint32_t elem_size) {
    if (s->ndim == 0 || s->strides[s->ndim - 1] != 1) {
        o_slice_pack(dst, src_base, s, elem_size);
        return;
    }
    const uint64_t run = s->sizes[s->ndim - 1];
    const uint64_t len = o_slice_len(s);
    if (run == 0 || len == 0) return;
    const int64_t rows = (int64_t)(len / run);
    /* long runs are cut into 1 MiB pieces so that a slice of few rows still uses every core */
    const uint64_t piece = (1u << 20) / elem_size ? (1u << 20) / elem_size : 1;
    const int64_t per_row = (int64_t)((run + piece - 1) / piece);
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < rows * per_row; t++) {
        const uint64_t r = (uint64_t)(t / per_row), first = (uint64_t)(t % per_row) * piece;
        const uint64_t n = run - first < piece ? run - first : piece;
        uint64_t loc;
        o_slice_get(s, r * run, &loc);
        memcpy((char*)dst + (r * run + first) * elem_size,
               (const char*)src_base + (loc + first) * elem_size, n * elem_size);
    }
}

void o_reduce_bf16_mt(uint16_t* out, const uint16_t* const* in, uint32_t n, uint64_t numel, int op) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)numel; i++) {
        float acc = bf16_to_f32(in[0][i]);
        for (uint32_t r = 1; r < n; r++) acc += bf16_to_f32(in[r][i]);
        if (op == 4) acc = acc / (float)n;
        out[i] = f32_to_bf16_rne(acc);
    }
}

void o_reduce_f32_mt(float* out, const float* const* in, uint32_t n, uint64_t numel, int op) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)numel; i++) {
        float acc = in[0][i];
        for (uint32_t r = 1; r < n; r++) acc += in[r][i];
        if (op == 4) acc = acc / (float)n;
        out[i] = acc;
    }
}

int o_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ====================================================================================
 * Device-initiated RDMA: work-queue and completion-queue entries (mlx5 wire format).
 *
 * Restates rdmaxcel-sys/src/rdmaxcel.cu:82-93 (db_ring), :139-160 (recv_wqe), :201-245
 * (send_wqe) and :292-326 (cqe_poll) over ordinary host memory.  The segment layouts
 * come from rdma-core's <infiniband/mlx5dv.h> (system package rdma-core-devel, no
 * version pinned, README.md:83; absent from the reference tree and from this image),
 * whose published layout is, in bytes, every multi-byte field big-endian:
 *
 *   mlx5_wqe_ctrl_seg  (16): 0-3 opmod_idx_opcode, 4-7 qpn_ds, 8 signature, 9-10 reserved
 *                            (dci_stream_channel_id), 11 fm_ce_se, 12-15 imm
 *                            (the reference repeats it at rdmaxcel-sys/src/lib.rs:22-31)
 *   mlx5_wqe_raddr_seg (16): 0-7 raddr, 8-11 rkey, 12-15 reserved
 *   mlx5_wqe_data_seg  (16): 0-3 byte_count, 4-7 lkey, 8-15 addr
 *   MLX5_SEND_WQE_SHIFT 6 (64-byte send WQE slots), MLX5_RCV_DBR 0, MLX5_SND_DBR 1,
 *   MLX5_WQE_CTRL_CQ_UPDATE 8 (2 << 2), MLX5_WQE_CTRL_SOLICITED 2 (1 << 1)
 *   mlx5_cqe64: byte_cnt big-endian at byte 44, op_own in the last byte
 *               (opcode in the upper 4 bits, ownership in bit 0)
 *
 * Pinning: the reference holds no byte vector of a WQE or CQE (its tests need two NICs,
 * monarch_rdma/src/rdma_manager_actor_tests.rs:396-600): PARITY UNPINNED in the reference.
 * Pinned here by known-answer bytes derived by hand from the layout above
 * (tests/test_oracle_rdmaxcel.py).
 *
 * The functions below assemble every field byte by byte, most significant byte first, rather
 * than swapping words, so that they share no code shape with the product's kernels.
 * ==================================================================================== */
typedef struct { /* wqe_params_t, rdmaxcel-sys/src/rdmaxcel.h:26-39 */
    uint64_t laddr;
    uint32_t lkey;
    uint64_t length;
    uint64_t wr_id;
    uint8_t signaled;
    uint32_t op_type;
    uint64_t raddr;
    uint32_t rkey;
    uint32_t qp_num;
    uint8_t* buf;
    uint32_t* dbrec;
    uint32_t wqe_cnt;
} o_wqe_params_t;

typedef struct { /* cqe_poll_params_t, rdmaxcel-sys/src/rdmaxcel.h:42-48 */
    uint8_t* cqe_buf;
    uint32_t cqe_size;
    uint32_t consumer_index;
    uint32_t cqe_cnt;
    uint32_t* dbrec;
} o_cqe_poll_params_t;

static void put_be32(uint8_t* p, uint32_t v) {
    p[0] = (uint8_t)(v >> 24);
    p[1] = (uint8_t)(v >> 16);
    p[2] = (uint8_t)(v >> 8);
    p[3] = (uint8_t)v;
}
static void put_be64(uint8_t* p, uint64_t v) {
    put_be32(p, (uint32_t)(v >> 32));
    put_be32(p + 4, (uint32_t)v);
}

/* rdmaxcel.cu:82-93: eight 64-bit words, lowest address first. */
void o_db_ring(void* dst, const void* src) {
    for (int i = 0; i < 8; i++) memcpy((uint8_t*)dst + 8 * i, (const uint8_t*)src + 8 * i, 8);
}

/* rdmaxcel.cu:139-160: one data segment at params.buf itself (the caller addresses the slot);
 * length and wr_id + 1 are cut to 32 bits by the 32-bit swap they are passed to (:148,:159). */
void o_recv_wqe(const o_wqe_params_t* p) {
    uint8_t seg[16];
    put_be32(seg + 0, (uint32_t)p->length);
    put_be32(seg + 4, p->lkey);
    put_be64(seg + 8, p->laddr);
    memcpy(p->buf, seg, 16);
    put_be32((uint8_t*)&p->dbrec[0], (uint32_t)(p->wr_id + 1));
}

/* rdmaxcel.cu:201-245.  idx is wr_id cut to 32 bits (:206); the slot is idx & (wqe_cnt - 1)
 * (:207) at 64 bytes per slot (:234); opmod_idx_opcode = (idx << 8) | op_type in 32 bits, so
 * idx bits 24-31 fall off and bits 16-23 land in the opmod byte (:214); qpn_ds = qp_num << 8 | 3
 * (:220); the three segments are zero-initialised (:202-204), so signature, the reserved bytes,
 * imm and the raddr segment's last word are written as zeros; the send doorbell record takes
 * (idx + 1) & 0xFFFFFF (:244). */
void o_send_wqe(const o_wqe_params_t* p) {
    const uint32_t idx = (uint32_t)p->wr_id;
    const uint32_t slot = idx & (p->wqe_cnt - 1u);
    uint8_t wqe[48];
    memset(wqe, 0, sizeof wqe);
    put_be32(wqe + 0, (idx << 8) | p->op_type);
    put_be32(wqe + 4, (p->qp_num << 8) | 3u);
    wqe[11] = p->signaled ? (uint8_t)(8 | 2) : 0;
    put_be64(wqe + 16, p->raddr);
    put_be32(wqe + 24, p->rkey);
    put_be32(wqe + 32, (uint32_t)p->length);
    put_be32(wqe + 36, p->lkey);
    put_be64(wqe + 40, p->laddr);
    memcpy(p->buf + ((uint64_t)slot << 6), wqe, 48);
    put_be32((uint8_t*)&p->dbrec[1], (idx + 1u) & 0xFFFFFFu);
}

/* rdmaxcel.cu:292-326: one look at the entry consumer_index & (cqe_cnt - 1).  Software owns it
 * when bit 0 of op_own equals the lap parity (consumer_index / cqe_cnt) & 1 and the opcode is not
 * 0xF (:310-311); an owned entry whose opcode has either of its two upper bits set is an error
 * (:314-315, -2), otherwise *byte_cnt receives the big-endian word at byte 44 as a signed 32-bit
 * value (:318); both owned cases store (consumer_index + 1) & 0xFFFFFF big-endian at dbrec[0]
 * (:319-324).  An entry that is not owned leaves *byte_cnt and the record alone. */
void o_cqe_poll(int32_t* byte_cnt, const o_cqe_poll_params_t* p) {
    const uint32_t idx = p->consumer_index;
    const uint8_t* cqe = p->cqe_buf + (uint64_t)(idx & (p->cqe_cnt - 1u)) * p->cqe_size;
    const uint8_t op_own = cqe[p->cqe_size - 1];
    const uint8_t opcode = (uint8_t)(op_own >> 4);
    const int owned = ((op_own & 1u) == ((idx / p->cqe_cnt) & 1u)) && opcode != 0xF;
    if (!owned) return;
    if ((opcode & 0xC) == 0) {
        *byte_cnt = (int32_t)(((uint32_t)cqe[44] << 24) | ((uint32_t)cqe[45] << 16) | ((uint32_t)cqe[46] << 8) | cqe[47]);
    } else {
        *byte_cnt = -2;
    }
    put_be32((uint8_t*)&p->dbrec[0], (idx + 1u) & 0xFFFFFFu);
}
