// Reduce (sum / avg / prod / max / min) over the chunks one GPU holds, with and without scatter.
//
// HBM-bound: (n + 1) * numel * sizeof(T) bytes per call.  Each lane moves 16 bytes per
// input per step; all n loads of a step are issued before the first add so that a
// wavefront keeps n KiB in flight.  Accumulation is fp32 (fp64 for f64) in rank order,
// rounded once at the end; out may alias in[0] because a lane reads every input of its
// own elements before it writes them.
#include <type_traits>

#include "mhip_device.h"

namespace mhip {

constexpr int kMaxInputs = 64;
constexpr int kMaxOutputs = 16;

struct ReduceArgs {
    void* out;
    const void* in[kMaxInputs];
    uint64_t numel;
    uint32_t n;
    float scale;   // 1/n when n is a power of two and op is Avg (exact), else 0
    float divisor; // n as a float
    uint32_t xcd_contiguous;  // kMap*: which chunk a workgroup takes, see inputs_alias()
    uint32_t op;              // MHIP_OP_*, read by the kGeneric kernels only
};

// How a kernel combines: Sum and Avg (the hot ops) are compiled as plain adds; Prod / Max / Min share one
// instantiation per type that switches on the (wave-uniform) op in the arguments.
enum : int { kSum = 0, kAvg = 1, kGeneric = 2 };

// ---- per-type vector traits: 16 bytes <-> accumulator lanes ----
template <typename T> struct Vec;

template <> struct Vec<float> {
    static constexpr int V = 4;
    using acc_t = float;
    __device__ static void widen(const uint4& r, acc_t* a) {
        a[0] = __uint_as_float(r.x); a[1] = __uint_as_float(r.y);
        a[2] = __uint_as_float(r.z); a[3] = __uint_as_float(r.w);
    }
    __device__ static uint4 narrow(const acc_t* a) {
        return make_uint4(__float_as_uint(a[0]), __float_as_uint(a[1]), __float_as_uint(a[2]), __float_as_uint(a[3]));
    }
    __device__ static acc_t widen1(const void* p, uint64_t i) { return static_cast<const float*>(p)[i]; }
    __device__ static void narrow1(void* p, uint64_t i, acc_t v) { static_cast<float*>(p)[i] = v; }
};

struct bf16_tag {};
template <> struct Vec<bf16_tag> {
    static constexpr int V = 8;
    using acc_t = float;
    __device__ static void widen(const uint4& r, acc_t* a) {
        a[0] = bf16_lo(r.x); a[1] = bf16_hi(r.x); a[2] = bf16_lo(r.y); a[3] = bf16_hi(r.y);
        a[4] = bf16_lo(r.z); a[5] = bf16_hi(r.z); a[6] = bf16_lo(r.w); a[7] = bf16_hi(r.w);
    }
    __device__ static uint4 narrow(const acc_t* a) {
        return make_uint4(pack_bf16x2(a[0], a[1]), pack_bf16x2(a[2], a[3]), pack_bf16x2(a[4], a[5]),
                          pack_bf16x2(a[6], a[7]));
    }
    __device__ static acc_t widen1(const void* p, uint64_t i) {
        return __uint_as_float((uint32_t) static_cast<const uint16_t*>(p)[i] << 16);
    }
    __device__ static void narrow1(void* p, uint64_t i, acc_t v) {
        static_cast<uint16_t*>(p)[i] = (uint16_t)f32_to_bf16_bits(v);
    }
};

template <> struct Vec<_Float16> {
    static constexpr int V = 8;
    using acc_t = float;
    union U { uint4 r; _Float16 h[8]; };
    __device__ static void widen(const uint4& r, acc_t* a) {
        U u; u.r = r;
#pragma unroll
        for (int k = 0; k < 8; ++k) a[k] = (float)u.h[k];
    }
    __device__ static uint4 narrow(const acc_t* a) {
        U u;
#pragma unroll
        for (int k = 0; k < 8; ++k) u.h[k] = (_Float16)a[k];
        return u.r;
    }
    __device__ static acc_t widen1(const void* p, uint64_t i) { return (float)static_cast<const _Float16*>(p)[i]; }
    __device__ static void narrow1(void* p, uint64_t i, acc_t v) { static_cast<_Float16*>(p)[i] = (_Float16)v; }
};

template <> struct Vec<double> {
    static constexpr int V = 2;
    using acc_t = double;
    union U { uint4 r; double d[2]; };
    __device__ static void widen(const uint4& r, acc_t* a) { U u; u.r = r; a[0] = u.d[0]; a[1] = u.d[1]; }
    __device__ static uint4 narrow(const acc_t* a) { U u; u.d[0] = a[0]; u.d[1] = a[1]; return u.r; }
    __device__ static acc_t widen1(const void* p, uint64_t i) { return static_cast<const double*>(p)[i]; }
    __device__ static void narrow1(void* p, uint64_t i, acc_t v) { static_cast<double*>(p)[i] = v; }
};

// integers: wrapping sum in the unsigned type of the same width
template <typename UT> struct IntVec {
    static constexpr int V = 16 / sizeof(UT);
    using acc_t = UT;
    union U { uint4 r; UT e[V]; };
    __device__ static void widen(const uint4& r, acc_t* a) {
        U u; u.r = r;
#pragma unroll
        for (int k = 0; k < V; ++k) a[k] = u.e[k];
    }
    __device__ static uint4 narrow(const acc_t* a) {
        U u;
#pragma unroll
        for (int k = 0; k < V; ++k) u.e[k] = a[k];
        return u.r;
    }
    __device__ static acc_t widen1(const void* p, uint64_t i) { return static_cast<const UT*>(p)[i]; }
    __device__ static void narrow1(void* p, uint64_t i, acc_t v) { static_cast<UT*>(p)[i] = v; }
};
template <> struct Vec<uint8_t> : IntVec<uint8_t> {};
template <> struct Vec<uint32_t> : IntVec<uint32_t> {};
template <> struct Vec<uint64_t> : IntVec<uint64_t> {};
// signed flavours: Max / Min compare them as signed, Prod wraps like Sum does
template <> struct Vec<int8_t> : IntVec<int8_t> {};
template <> struct Vec<int32_t> : IntVec<int32_t> {};
template <> struct Vec<int64_t> : IntVec<int64_t> {};

// acc (op) x.  Max / Min keep the accumulator on ties (so the first of +0 / -0 in member order wins) and skip
// NaN operands unless every operand is NaN, which is what ncclMax / ncclMin compute with fmaxf / fminf
// (the op numbering is torch-sys-cuda/src/nccl.rs:285-292; NCCL itself is not part of the reference tree).
// Integer Prod wraps (computed in the unsigned type of the same width).
template <int MODE, typename A>
__device__ __forceinline__ A combine(A acc, A x, uint32_t op) {
    if constexpr (MODE != kGeneric) {
        return acc + x;
    } else if constexpr (std::is_floating_point<A>::value) {
        switch (op) {
            case MHIP_OP_PROD: return acc * x;
            case MHIP_OP_MAX: return (x > acc || acc != acc) ? x : acc;
            case MHIP_OP_MIN: return (x < acc || acc != acc) ? x : acc;
            default: return acc + x;
        }
    } else {
        using UA = typename std::make_unsigned<A>::type;
        switch (op) {
            case MHIP_OP_PROD: return (A)(UA)((UA)acc * (UA)x);
            case MHIP_OP_MAX: return x > acc ? x : acc;
            case MHIP_OP_MIN: return x < acc ? x : acc;
            default: return (A)(UA)((UA)acc + (UA)x);
        }
    }
}

// The same over the V lanes of one vector, with the (wave-uniform) op tested once per vector instead of once per
// element: the element loops of Prod / Max / Min are then as tight as the adds of Sum.
template <int MODE, int V, typename A>
__device__ __forceinline__ void combine_vec(A* acc, const A* x, uint32_t op) {
    if constexpr (MODE != kGeneric) {
#pragma unroll
        for (int k = 0; k < V; ++k) acc[k] = acc[k] + x[k];
    } else {
        switch (op) {
            case MHIP_OP_PROD:
#pragma unroll
                for (int k = 0; k < V; ++k) acc[k] = combine<kGeneric>(acc[k], x[k], MHIP_OP_PROD);
                break;
            case MHIP_OP_MAX:
#pragma unroll
                for (int k = 0; k < V; ++k) acc[k] = combine<kGeneric>(acc[k], x[k], MHIP_OP_MAX);
                break;
            case MHIP_OP_MIN:
#pragma unroll
                for (int k = 0; k < V; ++k) acc[k] = combine<kGeneric>(acc[k], x[k], MHIP_OP_MIN);
                break;
            default:
#pragma unroll
                for (int k = 0; k < V; ++k) acc[k] = combine<kGeneric>(acc[k], x[k], MHIP_OP_SUM);
                break;
        }
    }
}

template <typename A> __device__ __forceinline__ A finish(A acc, bool avg, float scale, float divisor) {
    if constexpr (std::is_same<A, float>::value) {
        if (avg) return scale != 0.0f ? acc * scale : acc / divisor;
    } else if constexpr (std::is_same<A, double>::value) {
        if (avg) return acc / (double)divisor;
    }
    return acc;
}

// K more inputs, in[r] .. in[r + K - 1], added to acc in that order: all K loads are issued before the first add.
template <typename T, int K, int MODE>
__device__ __forceinline__ void add_group(typename Vec<T>::acc_t* acc, const void* const* in, uint32_t r, uint64_t v, uint32_t op) {
    using VT = Vec<T>;
    uint4 raw[K];
#pragma unroll
    for (int j = 0; j < K; ++j) raw[j] = load16_unaligned(static_cast<const char*>(in[r + j]) + v * 16);
#pragma unroll
    for (int j = 0; j < K; ++j) {
        typename VT::acc_t x[VT::V];
        VT::widen(raw[j], x);
        combine_vec<MODE, VT::V>(acc, x, op);
    }
}

// N > 0: compile-time input count (all loads hoisted); N == 0: runtime count, groups of 8 and one last group of
// what is left, each with its loads hoisted (5 bf16 inputs of 48 MiB: 0.77 of peak when the last four were loaded
// and added one after the other).
//
// Workgroups are 128 lanes and the grid covers the buffer in one pass (one 16-byte
// vector per lane): on MI355X this shape streams ~7% faster than 256-lane groups or a
// persistent grid-stride loop (5.99 vs 5.56 TB/s for 8 bf16 inputs of 48 MiB).
constexpr int kReduceThreads = 128;

// Workgroup i runs on XCD i mod 8, and a workgroup covers 2 KiB of every input, so with the
// plain mapping one XCD only ever touches addresses that agree modulo 16 KiB.  That is the
// fastest arrangement when the inputs themselves sit at different 4 KiB phases of 16 KiB (what
// mhip_staging_slot_pitch arranges): 8 x 48 MiB bf16 at 70.6 us.  When more than half of the
// inputs share a phase (slots packed back to back, power-of-two slabs of one tensor) it is the
// slowest (75.6 us), and handing each XCD one contiguous eighth of the index space instead is
// better (73.1 us; the fp32 mesh-dim reduce+scatter over 32 MiB slabs 105 -> 96 us).  Better still for
// the plain reduce is to leave workgroup i in its own group of 8 consecutive chunks and advance the chunk it
// takes there by one per group: consecutive workgroups still cover consecutive memory, and an XCD meets all
// eight 2 KiB phases of 16 KiB in turn (8 separately allocated bf16 inputs of 48 MiB, the three mappings in
// turn on one GPU: plain 0.759, contiguous eighths 0.769, rotated 0.785 of peak; the reduce + scatter does
// better with the eighths, 0.78 against 0.75).  The host looks at the input addresses and picks the mapping
// per launch.
static bool inputs_alias(const void* const* in, uint32_t n) {
    if (n < 4) return false;
    uint32_t count[4] = {0, 0, 0, 0};
    for (uint32_t r = 0; r < n; ++r) ++count[((uintptr_t)in[r] >> 12) & 3u];
    uint32_t most = 0;
    for (uint32_t c : count) most = c > most ? c : most;
    return most * 2 > n;
}

enum : uint32_t { kMapPlain = 0, kMapEighths = 1, kMapRotated = 2 };

__device__ __forceinline__ uint32_t xcd_rotated_block() {
    if (blockIdx.x >= (gridDim.x & ~7u)) return blockIdx.x;  // the last, partial group of 8 keeps its order
    return (blockIdx.x & ~7u) | ((blockIdx.x + (blockIdx.x >> 3)) & 7u);
}

__device__ __forceinline__ uint32_t xcd_contiguous_block() {
    const uint32_t per = gridDim.x / 8;  // blocks past the last whole group of 8 keep their index
    return blockIdx.x < per * 8 ? (blockIdx.x & 7u) * per + (blockIdx.x >> 3) : blockIdx.x;
}

template <typename T, int N, int MODE>
__global__ __launch_bounds__(kReduceThreads) void reduce_kernel(ReduceArgs a) {
    using VT = Vec<T>;
    using acc_t = typename VT::acc_t;
    constexpr int V = VT::V;
    const uint64_t nvec = a.numel / V;
    const uint64_t stride = (uint64_t)gridDim.x * kReduceThreads;
    const uint32_t bid = a.xcd_contiguous == kMapRotated ? xcd_rotated_block() : a.xcd_contiguous ? xcd_contiguous_block() : blockIdx.x;
    for (uint64_t v = (uint64_t)bid * kReduceThreads + threadIdx.x; v < nvec; v += stride) {
        acc_t acc[V];
        if constexpr (N > 0) {
            uint4 raw[N];
#pragma unroll
            for (int r = 0; r < N; ++r) raw[r] = load16_unaligned(static_cast<const char*>(a.in[r]) + v * 16);
            VT::widen(raw[0], acc);
#pragma unroll
            for (int r = 1; r < N; ++r) {
                acc_t x[V];
                VT::widen(raw[r], x);
                combine_vec<MODE, V>(acc, x, a.op);
            }
        } else {
            VT::widen(load16_unaligned(static_cast<const char*>(a.in[0]) + v * 16), acc);
            uint32_t r = 1;
            for (; r + 8 <= a.n; r += 8) add_group<T, 8, MODE>(acc, a.in, r, v, a.op);
            switch (a.n - r) {  // wave-uniform
                case 7: add_group<T, 7, MODE>(acc, a.in, r, v, a.op); break;
                case 6: add_group<T, 6, MODE>(acc, a.in, r, v, a.op); break;
                case 5: add_group<T, 5, MODE>(acc, a.in, r, v, a.op); break;
                case 4: add_group<T, 4, MODE>(acc, a.in, r, v, a.op); break;
                case 3: add_group<T, 3, MODE>(acc, a.in, r, v, a.op); break;
                case 2: add_group<T, 2, MODE>(acc, a.in, r, v, a.op); break;
                case 1: add_group<T, 1, MODE>(acc, a.in, r, v, a.op); break;
                default: break;
            }
        }
#pragma unroll
        for (int k = 0; k < V; ++k) acc[k] = finish(acc[k], MODE == kAvg, a.scale, a.divisor);
        store16_writethrough(static_cast<char*>(a.out) + v * 16, VT::narrow(acc));
    }
    // ragged tail: fewer than V elements, one lane each
    if (blockIdx.x == 0) {
        const uint64_t i = nvec * V + threadIdx.x;
        if (threadIdx.x < V && i < a.numel) {
            acc_t acc = VT::widen1(a.in[0], i);
            uint32_t r = 1;
            for (; r + 8 <= a.n; r += 8) {  // eight loads in flight, as in the body
                acc_t x[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) x[j] = VT::widen1(a.in[r + j], i);
#pragma unroll
                for (int j = 0; j < 8; ++j) acc = combine<MODE>(acc, x[j], a.op);
            }
            for (; r < a.n; ++r) acc = combine<MODE>(acc, VT::widen1(a.in[r], i), a.op);
            VT::narrow1(a.out, i, finish(acc, MODE == kAvg, a.scale, a.divisor));
        }
    }
}

// ---------------- reduce + scatter ----------------

struct ScatterArgs {
    void* outs[kMaxOutputs];
    uint64_t out_offset[kMaxOutputs];  // units into the reduced tensor's index space
    const void* in[kMaxInputs];
    uint64_t total;                    // units per output
    uint64_t in_offset;                // units
    uint32_t n_in;
    uint32_t n_out;                    // outputs handled by this launch
    float scale;
    float divisor;
    uint32_t xcd_contiguous;           // see inputs_alias()
    uint32_t op;                       // MHIP_OP_*, read by the kGeneric kernels only
    DimsArg out_dims;                  // packed output index -> reduced-tensor index
    DimsArg in_dims;                   // reduced-tensor index -> input memory
};

// VEC: a unit is 16 bytes (V elements) and never straddles a row of either view.
// D: number of dimensions (outside the run) both decodes are compiled for; shorter views
// are padded on the host.  D < 0 reads the counts from the arguments.
template <typename T, bool VEC, int MODE, bool WIDE, int D>
__global__ __launch_bounds__(kReduceThreads) void reduce_scatter_kernel(ScatterArgs a) {
    using VT = Vec<T>;
    using acc_t = typename VT::acc_t;
    constexpr int V = VT::V;
    // The output index is the FASTEST-varying part of the workgroup id: workgroups that run
    // side by side handle the same position of neighbouring outputs, which for column-block
    // scatters are neighbouring segments of the same input rows (sequential HBM reads).
    // (Rotating k by the tile number, so that an output is not pinned to one XCD, was
    // measured and does not help: -6% on flat chunks, +0.5% on column blocks.)
    const uint32_t nk = a.n_out;
    const uint32_t bid = a.xcd_contiguous ? xcd_contiguous_block() : blockIdx.x;
    const uint64_t tile0 = bid / nk;
    const uint32_t k = bid % nk;
    const uint64_t stride = (uint64_t)(gridDim.x / nk) * kReduceThreads;
    for (uint64_t t = tile0 * kReduceThreads + threadIdx.x; t < a.total; t += stride) {
        uint64_t col;
        const uint64_t i = a.out_offset[k] + decode<WIDE, D>(a.out_dims, t, &col);
        const uint64_t loc = a.in_offset + decode<WIDE, D>(a.in_dims, i, &col);
        if constexpr (VEC) {
            acc_t acc[V];
            VT::widen(load16_unaligned(static_cast<const char*>(a.in[0]) + loc * 16), acc);
            uint32_t g = 1;
            for (; g + 7 <= a.n_in; g += 7) {
                uint4 raw[7];
#pragma unroll
                for (int j = 0; j < 7; ++j) raw[j] = load16_unaligned(static_cast<const char*>(a.in[g + j]) + loc * 16);
#pragma unroll
                for (int j = 0; j < 7; ++j) {
                    acc_t x[V];
                    VT::widen(raw[j], x);
                    combine_vec<MODE, V>(acc, x, a.op);
                }
            }
            for (; g < a.n_in; ++g) {
                acc_t x[V];
                VT::widen(load16_unaligned(static_cast<const char*>(a.in[g]) + loc * 16), x);
                combine_vec<MODE, V>(acc, x, a.op);
            }
#pragma unroll
            for (int e = 0; e < V; ++e) acc[e] = finish(acc[e], MODE == kAvg, a.scale, a.divisor);
            store16_writethrough(static_cast<char*>(a.outs[k]) + t * 16, VT::narrow(acc));
        } else {
            acc_t acc = VT::widen1(a.in[0], loc);
            for (uint32_t g = 1; g < a.n_in; ++g) acc = combine<MODE>(acc, VT::widen1(a.in[g], loc), a.op);
            VT::narrow1(a.outs[k], t, finish(acc, MODE == kAvg, a.scale, a.divisor));
        }
    }
}

// Element-granular views whose rows are still at least one 16-byte vector long (odd row lengths,
// odd offsets): the work is cut into V-element chunks of each output.  A chunk inside one output
// row is one vector; a chunk that straddles a row boundary is computed as two whole vectors, A
// ending at the row end and B starting the next row, which overlap the neighbouring chunks and
// write the same bits there (the sum order does not depend on the lane).  The vectors' loads carry no
// per-lane predicate (lanes without one read an aligned dummy, one address per wavefront).
// A vector that would cross a row of the INPUT view, and the last partial chunk, go element by
// element.  Against the purely scalar form: fp32 rows of 511 0.44 -> 0.68 of peak, bf16 rows of 1022 0.24 -> 0.66.
template <typename T, int MODE, bool WIDE, int D>
__global__ __launch_bounds__(kReduceThreads) void reduce_scatter_ragged_kernel(ScatterArgs a) {
    using VT = Vec<T>;
    using acc_t = typename VT::acc_t;
    constexpr int V = VT::V;
    constexpr int ES = 16 / V;
    const uint32_t nk = a.n_out;
    const uint32_t bid = a.xcd_contiguous ? xcd_contiguous_block() : blockIdx.x;
    const uint64_t tile0 = bid / nk;
    const uint32_t k = bid % nk;
    const uint64_t nchunks = (a.total + V - 1) / V;
    const uint64_t stride = (uint64_t)(gridDim.x / nk) * kReduceThreads;
    char* __restrict__ out = static_cast<char*>(a.outs[k]);

    auto one_element = [&](uint64_t t) {  // output element t of output k, all inputs, element loads
        uint64_t col;
        const uint64_t r = a.out_offset[k] + decode<WIDE, D>(a.out_dims, t, &col);
        const uint64_t loc = a.in_offset + decode<WIDE, D>(a.in_dims, r, &col);
        acc_t acc = VT::widen1(a.in[0], loc);
        for (uint32_t g = 1; g < a.n_in; ++g) acc = combine<MODE>(acc, VT::widen1(a.in[g], loc), a.op);
        VT::narrow1(out, t, finish(acc, MODE == kAvg, a.scale, a.divisor));
    };

    for (uint64_t c = tile0 * kReduceThreads + threadIdx.x; c < nchunks; c += stride) {
        const uint64_t first = c * V;
        if (a.total < (uint64_t)V) {  // an output shorter than one vector
            for (uint64_t t = first; t < a.total; ++t) one_element(t);
            continue;
        }
        uint64_t col;
        const uint64_t r0 = a.out_offset[k] + decode<WIDE, D>(a.out_dims, first, &col);
        const uint64_t rem = a.out_dims.run - col;
        uint64_t ta = first, ra = r0, tb = 0, rb = 0;
        bool do_b = false;
        if (rem < (uint64_t)V) {
            // the last chunk of the output ends its last row: vector A alone, ending where the output ends (one lane
            // summing the last elements one by one, input after input, cost a small launch 2-3 us)
            ta = first + rem - V;
            ra = r0 + rem - V;
            tb = first + rem;
            do_b = tb < a.total;
            if (do_b) rb = a.out_offset[k] + decode<WIDE, D>(a.out_dims, tb, &col);
        }
        uint64_t ca, cb;
        const uint64_t la = a.in_offset + decode<WIDE, D>(a.in_dims, ra, &ca);
        const uint64_t lb = a.in_offset + decode<WIDE, D>(a.in_dims, rb, &cb);  // rb == 0 when there is no B
        const bool a_vec = ca + V <= a.in_dims.run;
        const bool b_vec = cb + V <= a.in_dims.run;
        // Vector loads only from addresses known to hold a whole vector; the other lanes read the aligned vector
        // around the first element of each input (one address per wavefront).  Wavefronts in which no lane has a
        // second vector skip those loads altogether (fp32 rows of 8190: 0.74 -> 0.785 of peak, rows of 511 to 2045
        // +0.015, bf16 within 0.01 either way).
        const bool use_b = do_b && b_vec;
        auto src = [&](uint32_t g, bool use, uint64_t idx) -> const char* {
            const char* base = static_cast<const char*>(a.in[g]);
            return use ? base + idx * ES : reinterpret_cast<const char*>(((uintptr_t)base + a.in_offset * ES) & ~(uintptr_t)15);
        };
        acc_t acc_a[V], acc_b[V];
        if (__builtin_amdgcn_ballot_w64(use_b) != 0) {  // one branch for the whole wavefront
            VT::widen(load16_unaligned(src(0, a_vec, la)), acc_a);
            VT::widen(load16_unaligned(src(0, use_b, lb)), acc_b);
            uint32_t g = 1;
            for (; g + 4 <= a.n_in; g += 4) {
                uint4 raw_a[4], raw_b[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) raw_a[j] = load16_unaligned(src(g + j, a_vec, la));
#pragma unroll
                for (int j = 0; j < 4; ++j) raw_b[j] = load16_unaligned(src(g + j, use_b, lb));
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc_t x[V];
                    VT::widen(raw_a[j], x);
                    combine_vec<MODE, V>(acc_a, x, a.op);
                    VT::widen(raw_b[j], x);
                    combine_vec<MODE, V>(acc_b, x, a.op);
                }
            }
            for (; g < a.n_in; ++g) {
                acc_t x[V];
                VT::widen(load16_unaligned(src(g, a_vec, la)), x);
                combine_vec<MODE, V>(acc_a, x, a.op);
                VT::widen(load16_unaligned(src(g, use_b, lb)), x);
                combine_vec<MODE, V>(acc_b, x, a.op);
            }
        } else {
            VT::widen(load16_unaligned(src(0, a_vec, la)), acc_a);
            uint32_t g = 1;
            for (; g + 7 <= a.n_in; g += 7) {
                uint4 raw_a[7];
#pragma unroll
                for (int j = 0; j < 7; ++j) raw_a[j] = load16_unaligned(src(g + j, a_vec, la));
#pragma unroll
                for (int j = 0; j < 7; ++j) {
                    acc_t x[V];
                    VT::widen(raw_a[j], x);
                    combine_vec<MODE, V>(acc_a, x, a.op);
                }
            }
            for (; g < a.n_in; ++g) {
                acc_t x[V];
                VT::widen(load16_unaligned(src(g, a_vec, la)), x);
                combine_vec<MODE, V>(acc_a, x, a.op);
            }
        }
        if (a_vec) {
#pragma unroll
            for (int e = 0; e < V; ++e) acc_a[e] = finish(acc_a[e], MODE == kAvg, a.scale, a.divisor);
            store16_writethrough(out + ta * ES, VT::narrow(acc_a));
        } else {
            for (int e = 0; e < V; ++e) one_element(ta + e);
        }
        if (do_b) {
            if (b_vec) {
#pragma unroll
                for (int e = 0; e < V; ++e) acc_b[e] = finish(acc_b[e], MODE == kAvg, a.scale, a.divisor);
                store16_writethrough(out + tb * ES, VT::narrow(acc_b));
            } else {
                for (int e = 0; e < V; ++e) one_element(tb + e);
            }
        }
    }
}

// ---------------- host side ----------------

static uint32_t grid_for(uint64_t items) {
    // one pass over the data; the grid-stride loop only engages beyond the largest grid a launch can hold
    const uint64_t blocks = (items + kReduceThreads - 1) / kReduceThreads;
    const uint64_t cap = max_workgroups(kReduceThreads);
    return (uint32_t)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

static int check_dtype_op(int dtype, int op) {
    switch (dtype) {
        case MHIP_DTYPE_F8E5M2: case MHIP_DTYPE_F8E4M3FN: case MHIP_DTYPE_F8E5M2FNUZ: case MHIP_DTYPE_F8E4M3FNUZ:
            return MHIP_ERR_FLOAT8_REDUCTION;  // nccl.rs:474-476
        case MHIP_DTYPE_U8: case MHIP_DTYPE_I8: case MHIP_DTYPE_I32: case MHIP_DTYPE_I64:
            if (op == MHIP_OP_AVG) return MHIP_ERR_UNSUPPORTED_OP;
            break;
        case MHIP_DTYPE_F16: case MHIP_DTYPE_F32: case MHIP_DTYPE_F64: case MHIP_DTYPE_BF16:
            break;
        default:
            return MHIP_ERR_INVALID_DATA_TYPE;
    }
    if (op < MHIP_OP_SUM || op > MHIP_OP_AVG) return MHIP_ERR_UNSUPPORTED_OP;  // nccl.rs:285-292
    return MHIP_SUCCESS;
}

static int mode_of(int op) { return op == MHIP_OP_SUM ? kSum : op == MHIP_OP_AVG ? kAvg : kGeneric; }

static void avg_factors(uint32_t n, int op, float* scale, float* divisor) {
    *divisor = (float)n;
    *scale = (op == MHIP_OP_AVG && (n & (n - 1)) == 0) ? 1.0f / (float)n : 0.0f;
}

template <typename T, int MODE>
static void launch_reduce_n(const ReduceArgs& a, hipStream_t s) {
    const dim3 grid(grid_for(a.numel / Vec<T>::V)), block(kReduceThreads);
    if constexpr (MODE == kGeneric) {
        MHIP_LAUNCH((reduce_kernel<T, 0, MODE>), grid, block, 0, s, a);
    } else {
        switch (a.n) {
            case 1: MHIP_LAUNCH((reduce_kernel<T, 1, MODE>), grid, block, 0, s, a); break;
            case 2: MHIP_LAUNCH((reduce_kernel<T, 2, MODE>), grid, block, 0, s, a); break;
            case 3: MHIP_LAUNCH((reduce_kernel<T, 3, MODE>), grid, block, 0, s, a); break;
            case 4: MHIP_LAUNCH((reduce_kernel<T, 4, MODE>), grid, block, 0, s, a); break;
            case 5: MHIP_LAUNCH((reduce_kernel<T, 5, MODE>), grid, block, 0, s, a); break;
            case 6: MHIP_LAUNCH((reduce_kernel<T, 6, MODE>), grid, block, 0, s, a); break;
            case 7: MHIP_LAUNCH((reduce_kernel<T, 7, MODE>), grid, block, 0, s, a); break;
            case 8: MHIP_LAUNCH((reduce_kernel<T, 8, MODE>), grid, block, 0, s, a); break;
            default: MHIP_LAUNCH((reduce_kernel<T, 0, MODE>), grid, block, 0, s, a); break;
        }
    }
}

// T: the type Sum / Avg run in (integers as the unsigned type of their width); G: the type Prod / Max / Min run in
// (signed where the dtype is).
template <typename T, typename G = T>
static void launch_reduce(const ReduceArgs& a, int op, hipStream_t s) {
    switch (mode_of(op)) {
        case kSum: launch_reduce_n<T, kSum>(a, s); break;
        case kAvg: launch_reduce_n<T, kAvg>(a, s); break;
        default: launch_reduce_n<G, kGeneric>(a, s); break;
    }
}

template <typename T, bool VEC, int MODE>
static void launch_scatter_d(const ScatterArgs& a, dim3 grid, bool wide, int d, hipStream_t s) {
    const dim3 block(kReduceThreads);
    if (wide) { MHIP_LAUNCH((reduce_scatter_kernel<T, VEC, MODE, true, -1>), grid, block, 0, s, a); return; }
    if constexpr (MODE != kGeneric) {
        switch (d) {
            case 2: MHIP_LAUNCH((reduce_scatter_kernel<T, VEC, MODE, false, 2>), grid, block, 0, s, a); return;
            case 4: MHIP_LAUNCH((reduce_scatter_kernel<T, VEC, MODE, false, 4>), grid, block, 0, s, a); return;
            default: break;
        }
    }
    MHIP_LAUNCH((reduce_scatter_kernel<T, VEC, MODE, false, -1>), grid, block, 0, s, a);
}

template <typename T, int MODE>
static void launch_scatter_ragged(const ScatterArgs& a, dim3 grid, bool wide, int d, hipStream_t s) {
    const dim3 block(kReduceThreads);
    if (wide) { MHIP_LAUNCH((reduce_scatter_ragged_kernel<T, MODE, true, -1>), grid, block, 0, s, a); return; }
    if constexpr (MODE != kGeneric) {
        switch (d) {
            case 2: MHIP_LAUNCH((reduce_scatter_ragged_kernel<T, MODE, false, 2>), grid, block, 0, s, a); return;
            case 4: MHIP_LAUNCH((reduce_scatter_ragged_kernel<T, MODE, false, 4>), grid, block, 0, s, a); return;
            default: break;
        }
    }
    MHIP_LAUNCH((reduce_scatter_ragged_kernel<T, MODE, false, -1>), grid, block, 0, s, a);
}

template <typename T, int MODE>
static void launch_scatter_mode(const ScatterArgs& a, dim3 grid, bool vec, bool ragged, bool wide, int d, hipStream_t s) {
    if (ragged) launch_scatter_ragged<T, MODE>(a, grid, wide, d, s);
    else if (vec) launch_scatter_d<T, true, MODE>(a, grid, wide, d, s);
    else launch_scatter_d<T, false, MODE>(a, grid, wide, d, s);
}

template <typename T, typename G = T>
static void launch_scatter(const ScatterArgs& a, dim3 grid, bool vec, bool ragged, int op, bool wide, int d, hipStream_t s) {
    constexpr bool kFloat = std::is_floating_point<typename Vec<T>::acc_t>::value;
    const int mode = mode_of(op);
    if (mode == kGeneric) { launch_scatter_mode<G, kGeneric>(a, grid, vec, ragged, wide, d, s); return; }
    if constexpr (kFloat) {
        if (mode == kAvg) { launch_scatter_mode<T, kAvg>(a, grid, vec, ragged, wide, d, s); return; }
    }
    launch_scatter_mode<T, kSum>(a, grid, vec, ragged, wide, d, s);
}

}  // namespace mhip

using namespace mhip;

extern "C" {

uint32_t mhip_dtype_size(int dtype) {
    switch (dtype) {
        case MHIP_DTYPE_U8: case MHIP_DTYPE_I8: case MHIP_DTYPE_F8E5M2: case MHIP_DTYPE_F8E4M3FN:
        case MHIP_DTYPE_F8E5M2FNUZ: case MHIP_DTYPE_F8E4M3FNUZ: return 1;
        case MHIP_DTYPE_F16: case MHIP_DTYPE_BF16: return 2;
        case MHIP_DTYPE_I32: case MHIP_DTYPE_F32: return 4;
        case MHIP_DTYPE_I64: case MHIP_DTYPE_F64: return 8;
        default: return 0;
    }
}

int mhip_reduce(void* out, const void* const* in, uint32_t n, uint64_t numel, int dtype, int op,
                mhip_stream_t stream) {
    if (!in || n == 0) return MHIP_ERR_INVALID_ARGUMENT;
    if (int rc = check_dtype_op(dtype, op)) return rc;
    if (n > (uint32_t)kMaxInputs) return MHIP_ERR_TOO_MANY_INPUTS;
    if (numel == 0) return MHIP_SUCCESS;
    if (!out) return MHIP_ERR_UNDEFINED_TENSOR;
    const uint32_t esize = mhip_dtype_size(dtype);
    ReduceArgs a{};
    a.out = out;
    uintptr_t align = (uintptr_t)out;
    for (uint32_t r = 0; r < n; ++r) {
        if (!in[r]) return MHIP_ERR_UNDEFINED_TENSOR;
        a.in[r] = in[r];
        align |= (uintptr_t)in[r];
    }
    if (align & (esize - 1)) return MHIP_ERR_INVALID_ARGUMENT;  // not even element-aligned
    a.numel = numel;
    a.n = n;
    avg_factors(n, op, &a.scale, &a.divisor);
    a.xcd_contiguous = inputs_alias(in, n) ? kMapRotated : kMapPlain;
    a.op = (uint32_t)op;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    switch (dtype) {
        case MHIP_DTYPE_F32: launch_reduce<float>(a, op, hs); break;
        case MHIP_DTYPE_BF16: launch_reduce<bf16_tag>(a, op, hs); break;
        case MHIP_DTYPE_F16: launch_reduce<_Float16>(a, op, hs); break;
        case MHIP_DTYPE_F64: launch_reduce<double>(a, op, hs); break;
        case MHIP_DTYPE_U8: launch_reduce<uint8_t>(a, op, hs); break;
        case MHIP_DTYPE_I8: launch_reduce<uint8_t, int8_t>(a, op, hs); break;
        case MHIP_DTYPE_I32: launch_reduce<uint32_t, int32_t>(a, op, hs); break;
        case MHIP_DTYPE_I64: launch_reduce<uint64_t, int64_t>(a, op, hs); break;
        default: return MHIP_ERR_INVALID_DATA_TYPE;
    }
    return launch_status();
}

int mhip_reduce_scatter(void* const* outs, const mhip_slice_t* out_views, uint32_t n_out, const void* const* in,
                        const mhip_slice_t* in_view, uint64_t in_numel, uint32_t n_in, int dtype, int op,
                        mhip_stream_t stream) {
    if (!in || n_in == 0 || (n_out && (!outs || !out_views))) return MHIP_ERR_INVALID_ARGUMENT;
    if (int rc = check_dtype_op(dtype, op)) return rc;
    if (n_in > (uint32_t)kMaxInputs) return MHIP_ERR_TOO_MANY_INPUTS;
    const uint32_t esize = mhip_dtype_size(dtype);
    const uint32_t V = 16 / esize;

    // the reduced tensor's index space
    const uint64_t one = in_numel, unit_stride = 1;
    mhip_slice_t dense{0, 1, &one, &unit_stride};
    const mhip_slice_t& iv = in_view ? *in_view : dense;
    if (iv.ndim > MHIP_MAX_DIMS || (iv.ndim && (!iv.sizes || !iv.strides))) return MHIP_ERR_INVALID_ARGUMENT;
    if (int rc = validate_slice(iv.sizes, iv.ndim, iv.strides, iv.ndim)) return rc;
    if (!slice_fits_address_space(iv, esize)) return MHIP_ERR_INVALID_ARGUMENT;
    const uint64_t reduced_len = slice_len(iv);

    uintptr_t in_align = 0;
    for (uint32_t g = 0; g < n_in; ++g) {
        if (!in[g]) return MHIP_ERR_UNDEFINED_TENSOR;
        in_align |= (uintptr_t)in[g];
    }
    if (in_align & (esize - 1)) return MHIP_ERR_INVALID_ARGUMENT;

    for (uint32_t k = 0; k < n_out; ++k) {
        const mhip_slice_t& ov = out_views[k];
        if (ov.ndim > MHIP_MAX_DIMS || (ov.ndim && (!ov.sizes || !ov.strides))) return MHIP_ERR_INVALID_ARGUMENT;
        if (int rc = validate_slice(ov.sizes, ov.ndim, ov.strides, ov.ndim)) return rc;
        if (!slice_fits_address_space(ov, esize)) return MHIP_ERR_INVALID_ARGUMENT;
        const uint64_t len = slice_len(ov);
        if (len == 0) continue;
        if (!outs[k]) return MHIP_ERR_UNDEFINED_TENSOR;
        if ((uintptr_t)outs[k] & (esize - 1)) return MHIP_ERR_INVALID_ARGUMENT;
        uint64_t hi = ov.offset;
        for (uint32_t d = 0; d < ov.ndim; ++d) hi += (ov.sizes[d] - 1) * ov.strides[d];
        if (hi >= reduced_len) return MHIP_ERR_INPUT_SIZE_MISMATCH;  // view reaches outside the reduced tensor
    }

    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    float scale, divisor;
    avg_factors(n_in, op, &scale, &divisor);

    uint32_t k = 0;
    while (k < n_out) {
        if (slice_len(out_views[k]) == 0) { ++k; continue; }
        // Vector form: units of V elements on both views and 16-byte aligned pointers.
        // Slices are canonicalised with elem_size 1, i.e. in elements; the alignment mask
        // carries the pointers divided by the element size.
        uint32_t max_unit = V;
        CanonSlice oc, ic;
        uint32_t ou = 1, iu = 1;
        for (;;) {
            const uint64_t omask = ((uintptr_t)outs[k] / esize);
            const uint64_t imask = (in_align / esize) | 0;  // pointers only
            canonicalize(out_views[k], 1, omask, max_unit, &oc, &ou);
            canonicalize(iv, 1, imask, max_unit, &ic, &iu);
            if (max_unit == 1 || (ou == V && iu == V)) break;
            max_unit = 1;  // fall back to element granularity for both
        }
        // out view offsets are into the reduced index space: with unit u they must be
        // whole units too, which canonicalize guarantees by folding offset into the mask.
        const bool vec = max_unit == V;
        ScatterArgs a{};
        a.xcd_contiguous = inputs_alias(in, n_in);
        bool o32 = false, i32 = false;
        const int nd = oc.ndim > ic.ndim ? oc.ndim : ic.ndim;
        const int d = nd <= 2 ? 2 : (nd <= 4 ? 4 : -1);  // compiled decode depths
        if (!make_dims_arg(oc, &a.out_dims, &o32, d > 0 ? d : 0) || !make_dims_arg(ic, &a.in_dims, &i32, d > 0 ? d : 0))
            return MHIP_ERR_UNSUPPORTED_OP;
        // the output decode yields reduced-tensor indices that the input decode divides again
        const bool wide = !(o32 && i32 && ic.total < kFastDivLimit - 64);
        a.total = oc.total;
        a.in_offset = ic.offset;
        a.n_in = n_in;
        a.scale = scale;
        a.divisor = divisor;
        for (uint32_t g = 0; g < n_in; ++g) a.in[g] = in[g];
        a.outs[0] = outs[k];
        a.out_offset[0] = oc.offset;
        uint32_t nbatch = 1;
        while (k + nbatch < n_out && nbatch < (uint32_t)kMaxOutputs) {
            CanonSlice nc;
            uint32_t nu = 1;
            if (!canonicalize(out_views[k + nbatch], 1, (uintptr_t)outs[k + nbatch] / esize, max_unit, &nc, &nu)) break;
            if (nu != ou || !same_shape(oc, nc)) break;
            a.outs[nbatch] = outs[k + nbatch];
            a.out_offset[nbatch] = nc.offset;
            ++nbatch;
        }
        a.n_out = nbatch;
        // element-granular views with rows of at least one vector on both sides: V-element chunks
        const bool ragged = !vec && V > 1 && oc.run >= V && ic.run >= V;
        uint64_t tiles = grid_for(ragged ? (a.total + V - 1) / V : a.total);
        while (tiles > 1 && tiles * nbatch > max_workgroups(kReduceThreads)) tiles = (tiles + 1) / 2;  // grid-stride takes over
        dim3 grid((uint32_t)(tiles * nbatch));
        a.op = (uint32_t)op;
        switch (dtype) {
            case MHIP_DTYPE_F32: launch_scatter<float>(a, grid, vec, ragged, op, wide, d, hs); break;
            case MHIP_DTYPE_BF16: launch_scatter<bf16_tag>(a, grid, vec, ragged, op, wide, d, hs); break;
            case MHIP_DTYPE_F16: launch_scatter<_Float16>(a, grid, vec, ragged, op, wide, d, hs); break;
            case MHIP_DTYPE_F64: launch_scatter<double>(a, grid, vec, ragged, op, wide, d, hs); break;
            case MHIP_DTYPE_U8: launch_scatter<uint8_t>(a, grid, vec, ragged, op, wide, d, hs); break;
            case MHIP_DTYPE_I8: launch_scatter<uint8_t, int8_t>(a, grid, vec, ragged, op, wide, d, hs); break;
            case MHIP_DTYPE_I32: launch_scatter<uint32_t, int32_t>(a, grid, vec, ragged, op, wide, d, hs); break;
            case MHIP_DTYPE_I64: launch_scatter<uint64_t, int64_t>(a, grid, vec, ragged, op, wide, d, hs); break;
            default: return MHIP_ERR_INVALID_DATA_TYPE;
        }
        if (int rc = launch_status()) return rc;
        k += nbatch;
    }
    return MHIP_SUCCESS;
}

}  // extern "C"
