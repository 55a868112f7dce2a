// Device-side helpers shared by the kernel sources (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <tuple>
#include <utility>

#include "mhip_internal.h"

namespace mhip {

constexpr int kThreads = 256;  // 4 wavefronts of 64 lanes

// Kernel-argument form of a CanonSlice: row-major decode of a packed unit index
// into a unit offset in the strided tensor.
struct DimsArg {
    uint64_t run;                      // contiguous units per row
    uint64_t size[kMaxCanonDims];      // outermost first
    uint64_t stride[kMaxCanonDims];    // units
    FastDiv32 run_div;                 // valid in 32-bit mode only
    FastDiv32 size_div[kMaxCanonDims];
    int ndim;
};

// `pad_to` > 0 left-pads the dimension list with (size 1, stride 0) entries up to that many
// dimensions, so that a kernel compiled for a fixed count can decode shorter slices.
inline bool make_dims_arg(const CanonSlice& c, DimsArg* d, bool* fits32, int pad_to = 0) {
    if (c.ndim > kMaxCanonDims || pad_to > kMaxCanonDims) return false;
    const int nd = pad_to > c.ndim ? pad_to : c.ndim;
    const int lead = nd - c.ndim;
    d->run = c.run;
    d->ndim = nd;
    bool small = c.total < kFastDivLimit - 64 && c.run < kFastDivLimit;
    for (int k = 0; k < kMaxCanonDims; ++k) {
        const bool real = k >= lead && k < nd;
        d->size[k] = real ? c.dims[k - lead].size : 1;
        d->stride[k] = real ? c.dims[k - lead].stride : 0;
        if (d->size[k] >= kFastDivLimit) small = false;
    }
    if (small) {
        d->run_div = FastDiv32((uint32_t)c.run);
        for (int k = 0; k < kMaxCanonDims; ++k) d->size_div[k] = FastDiv32((uint32_t)d->size[k]);
    }
    *fits32 = small;
    return true;
}

// Unit offset of packed unit t, and its column within the row (for run-boundary tests).
// NDIM >= 0 fixes the number of dimensions outside the run at compile time (no loop, no
// kernel-argument loads inside the decode); NDIM < 0 reads it from the arguments.
template <bool WIDE, int NDIM = -1>
__device__ __forceinline__ uint64_t decode(const DimsArg& d, uint64_t t, uint64_t* col_out) {
    const int ndim = NDIM >= 0 ? NDIM : d.ndim;
    if (ndim == 0) {
        *col_out = t;  // one row: run == total
        return t;
    }
    uint64_t off;
    if constexpr (WIDE) {
        uint64_t row = t / d.run;
        uint64_t col = t - row * d.run;
        *col_out = col;
        off = col;
        for (int k = ndim - 1; k > 0; --k) {
            uint64_t q = row / d.size[k];
            off += (row - q * d.size[k]) * d.stride[k];
            row = q;
        }
        off += row * d.stride[0];
    } else {
        uint32_t row, col;
        d.run_div.divmod((uint32_t)t, row, col);
        *col_out = col;
        off = col;
        if constexpr (NDIM >= 0) {
#pragma unroll
            for (int k = NDIM - 1; k > 0; --k) {
                uint32_t q, r;
                d.size_div[k].divmod(row, q, r);
                off += (uint64_t)r * d.stride[k];
                row = q;
            }
        } else {
            for (int k = ndim - 1; k > 0; --k) {
                uint32_t q, r;
                d.size_div[k].divmod(row, q, r);
                off += (uint64_t)r * d.stride[k];
                row = q;
            }
        }
        off += (uint64_t)row * d.stride[0];
    }
    return off;
}

// `type` is the unit as a value; `mem` is what a pointer into tensor memory points to.  The strided side of a copy is
// only guaranteed byte-aligned up to the element size of the CALLER's tensor, which may be less than the unit (a view
// of 4-byte-granular shape that starts at an odd bf16 column), so units in memory carry no alignment assumption;
// gfx950 under the HSA runtime services such accesses in hardware.
template <int U> struct UnitType;
template <> struct UnitType<1> { using type = uint8_t; using mem = uint8_t; };
template <> struct UnitType<2> { using type = uint16_t; typedef uint16_t __attribute__((aligned(1))) mem; };
template <> struct UnitType<4> { using type = uint32_t; typedef uint32_t __attribute__((aligned(1))) mem; };
template <> struct UnitType<8> { using type = uint64_t; typedef uint64_t __attribute__((aligned(1))) mem; };
template <> struct UnitType<16> { using type = uint4; using mem = uint4; };

// 16-byte access at an address that is only known to be unit-aligned.  gfx950 under
// the HSA runtime services unaligned global dwordx4 accesses in hardware, and the
// compiler emits a single global_load/store_dwordx4 for these.
//
// All bulk traffic on this path is touched exactly once, so loads carry the non-temporal
// hint (the "nt" bit): streamed lines are not kept in L2 / Infinity Cache at the expense of
// each other.  On MI355X this is worth ~10-15% of HBM bandwidth for copy and reduce kernels.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 __attribute__((aligned(1))) u32x4_unaligned;
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef u32x2 __attribute__((aligned(1))) u32x2_unaligned;
typedef uint32_t __attribute__((aligned(1))) u32_unaligned;

__device__ __forceinline__ uint4 load16_unaligned(const void* p) {
    const u32x4 v = __builtin_nontemporal_load(static_cast<const u32x4_unaligned*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint4 load16_aligned(const void* p) {
    const u32x4 v = __builtin_nontemporal_load(static_cast<const u32x4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void store16_unaligned(void* p, const uint4& v) {
    const u32x4 w = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(w, static_cast<u32x4_unaligned*>(p));
}
__device__ __forceinline__ void store16_aligned(void* p, const uint4& v) {
    const u32x4 w = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(w, static_cast<u32x4*>(p));
}
__device__ __forceinline__ void store8_unaligned(void* p, uint32_t a, uint32_t b) {
    const u32x2 w = {a, b};
    __builtin_nontemporal_store(w, static_cast<u32x2_unaligned*>(p));
}
// Write-through store (system-scope policy bit sc1, no nt) for kernels whose output is a
// small share of the traffic next to a wide read stream: on MI355X the 8-input bf16 reduce
// takes 71.6 us with these against 74.1 us with nt stores and 75.8 us with plain stores.
// It is the wrong choice where stores are a large or ragged share (fp8 dequant-accumulate
// into tensors: 1.68 ms vs 1.23 ms with nt), so only the reduce kernels use it.
//
// The store is inline assembly, so the compiler does not know that it is a store of more than 64 bits.  On gfx940 and
// later a vector-ALU write to the data registers of such a store needs TWO wait states after it; the compiler inserts
// them for its own stores only.  Without them the instruction scheduled right after the asm can overwrite the first
// data register before the store has read it (seen as a stray loop counter or LDS address in the first dword of a
// stored vector; one wait state cured the 4-byte transposing kernel and not the 1-byte one, whose next instruction
// is the address computation of the following LDS read).  s_nop 1 is two wait states, two issue cycles per store.
__device__ __forceinline__ void store16_writethrough_raw(void* p, const u32x4& w) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(w) : "memory");
}
__device__ __forceinline__ void store16_writethrough(void* p, const uint4& v) {
    const u32x4 w = {v.x, v.y, v.z, v.w};
    store16_writethrough_raw(p, w);
}
__device__ __forceinline__ uint32_t load4_unaligned(const void* p) {
    return __builtin_nontemporal_load(static_cast<const u32_unaligned*>(p));
}

// ---- aligned loads of a byte range that is not 16-byte aligned ----
// Unaligned 128-bit loads work on gfx950 but are not free: a 48 MiB copy whose source is 2 bytes
// off takes 19.4 us against 16.7 us aligned, and the fused fp8 quantiser loses 8% on buckets whose
// tensors start at odd element offsets.  Where the memory around the range may be read, a wavefront
// loads the enclosing aligned vectors instead and shifts the bytes into place: lane i needs the tail
// of its own vector and the head of lane i+1's, which a DPP wavefront shift delivers (lane 63 takes
// lane 0 of the next 1 KiB row), followed by a 128-bit funnel shift built from v_alignbyte.
__device__ __forceinline__ uint32_t wave_shl1(uint32_t v, uint32_t fill) {
    // lane i <- lane i + 1; lane 63 <- fill (wave-uniform)
    return (uint32_t)__builtin_amdgcn_update_dpp((int)fill, (int)v, 0x130, 0xF, 0xF, false);
}

// bytes [4 * D + r, 4 * D + r + 16) of the 32 bytes {a, b}
template <int D>
__device__ __forceinline__ uint4 funnel16(const uint4& a, const uint4& b, uint32_t r) {
    const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    return make_uint4(__builtin_amdgcn_alignbyte(w[D + 1], w[D], r), __builtin_amdgcn_alignbyte(w[D + 2], w[D + 1], r),
                      __builtin_amdgcn_alignbyte(w[D + 3], w[D + 2], r), __builtin_amdgcn_alignbyte(w[D + 4], w[D + 3], r));
}

// v[k] (k < N) are the lane's aligned vectors of N consecutive 1 KiB rows starting `shift` bytes before
// the wanted data, tail is the first vector after the last row (the same for all lanes).  Replaces every
// v[k] by the 16 wanted bytes.
template <int D, int N>
__device__ __forceinline__ void shift_rows(uint4 (&v)[N], const uint4& tail, uint32_t r) {
#pragma unroll
    for (int k = 0; k < N; ++k) {  // ascending: v[k + 1] is still untouched when row k needs its lane 0
        const uint4& after = k + 1 < N ? v[k + 1] : tail;
        uint4 next;
        next.x = wave_shl1(v[k].x, __builtin_amdgcn_readfirstlane(after.x));
        next.y = wave_shl1(v[k].y, __builtin_amdgcn_readfirstlane(after.y));
        next.z = wave_shl1(v[k].z, __builtin_amdgcn_readfirstlane(after.z));
        next.w = wave_shl1(v[k].w, __builtin_amdgcn_readfirstlane(after.w));
        v[k] = funnel16<D>(v[k], next, r);
    }
}

template <int N>
__device__ __forceinline__ void shift_rows_into_place(uint4 (&v)[N], const uint4& tail, uint32_t shift) {
    const uint32_t r = shift & 3u;
    switch (shift >> 2) {  // wave-uniform
        case 0: shift_rows<0, N>(v, tail, r); break;
        case 1: shift_rows<1, N>(v, tail, r); break;
        case 2: shift_rows<2, N>(v, tail, r); break;
        default: shift_rows<3, N>(v, tail, r); break;
    }
}

// bf16 <-> fp32.  Widening is exact; narrowing is round-to-nearest-even with NaN
// mapped to the canonical quiet NaN 0x7fc0 (what torch's CPU cast produces).
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    return (u & 0x7fffffffu) > 0x7f800000u ? 0x7fc0u : r;
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    return f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
}

// Makes the stream's device current for the duration of a launch and restores the
// caller's device afterwards, so entry points never depend on the current device.
class DeviceGuard {
public:
    explicit DeviceGuard(hipStream_t stream) {
        if (stream == nullptr) return;
        int dev = -1;
        if (hipStreamGetDevice(stream, &dev) != hipSuccess) { (void)hipGetLastError(); return; }
        if (hipGetDevice(&prev_) != hipSuccess) { prev_ = -1; return; }
        if (dev != prev_) {
            if (hipSetDevice(dev) == hipSuccess) restore_ = true;
        }
    }
    ~DeviceGuard() {
        if (restore_) (void)hipSetDevice(prev_);
    }
private:
    int prev_ = -1;
    bool restore_ = false;
};

// The library reads the process environment exactly once, while it is being loaded (runtime.cpp), never from an
// entry point: getenv races with a setenv of the host application on another thread, and a stray variable must not
// change which kernel a production process runs.  MONARCH_HIP_TUNING=1 at load time switches the tuning aids on: only
// then does tuning_env() look a variable up, at every call, so that an A/B sweep can switch variants inside one process.
extern const bool g_tuning;
extern const uint64_t g_max_launch_lanes;
inline const char* tuning_env(const char* name) { return g_tuning ? std::getenv(name) : nullptr; }

// The runtime forms the global size of a launch (workgroups x lanes) in 32 bits.  A launch of exactly
// 2^32 lanes is refused, and a larger one wraps silently: (2^26 + 1) workgroups of 64 lanes ran as ONE
// workgroup and reported success.  Every host launch therefore keeps its grid at or below this bound;
// grid-stride kernels clamp to it, one-shot kernels are launched in several pieces.
// With the tuning aids on, MONARCH_HIP_MAX_LAUNCH_LANES (read at load) lowers the bound: a test aid that drives
// small inputs through the clamped and multi-piece paths.
inline uint64_t max_launch_lanes() { return g_max_launch_lanes; }
inline uint64_t max_workgroups(uint32_t lanes) { return max_launch_lanes() / lanes; }

// Every kernel of the library is launched through MHIP_LAUNCH, which keeps the launch's own return value in a
// thread-local slot; launch_status() reports and clears that slot.  The thread's HIP "last error" is neither
// read nor reset, so an error an unrelated earlier call of the host application left there is not mistaken for a
// failed launch, and the application still finds it afterwards.
inline hipError_t& last_launch_error() {
    static thread_local hipError_t e = hipSuccess;
    return e;
}

template <typename... Params, typename... Args, size_t... I>
inline hipError_t launch_kernel_impl(void (*kernel)(Params...), dim3 grid, dim3 block, size_t lds_bytes, hipStream_t stream,
                                     std::index_sequence<I...>, Args&&... args) {
    std::tuple<Params...> values{static_cast<Params>(std::forward<Args>(args))...};  // converted to the kernel's own types
    void* ptrs[] = {static_cast<void*>(&std::get<I>(values))...};
    return hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, ptrs, lds_bytes, stream);
}

template <typename... Params, typename... Args>
inline void launch_kernel(void (*kernel)(Params...), dim3 grid, dim3 block, size_t lds_bytes, hipStream_t stream, Args&&... args) {
    static_assert(sizeof...(Params) == sizeof...(Args) && sizeof...(Params) > 0, "argument count");
    const hipError_t e = launch_kernel_impl(kernel, grid, block, lds_bytes, stream, std::index_sequence_for<Params...>{},
                                            std::forward<Args>(args)...);
    if (e != hipSuccess && last_launch_error() == hipSuccess) last_launch_error() = e;  // the first failure of several launches stays
}
#define MHIP_LAUNCH(kernel, grid, block, lds_bytes, stream, ...) \
    ::mhip::launch_kernel(kernel, grid, block, lds_bytes, stream, __VA_ARGS__)

inline int launch_status() {
    hipError_t& slot = last_launch_error();
    const hipError_t e = slot;
    slot = hipSuccess;
    return e == hipSuccess ? MHIP_SUCCESS : (int)e;
}

// Launches `wgs` workgroups of `lanes` lanes as one or more grids within the bound above:
// launch(first_workgroup, count) enqueues one piece, whose kernel adds first_workgroup to blockIdx.x.
// Pieces after the first start at a multiple of `multiple` workgroups.
template <typename F>
inline int launch_in_pieces(uint64_t wgs, uint32_t lanes, uint32_t multiple, F&& launch) {
    const uint64_t most = max_workgroups(lanes) / multiple * multiple;
    if (most == 0) return MHIP_ERR_INVALID_ARGUMENT;
    for (uint64_t first = 0; first < wgs; first += most) {
        launch(first, (uint32_t)(wgs - first < most ? wgs - first : most));
        if (int rc = launch_status()) return rc;
    }
    return MHIP_SUCCESS;
}

}  // namespace mhip
