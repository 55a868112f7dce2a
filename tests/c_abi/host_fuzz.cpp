// Host-only fuzz of the library's Slice code (slice_host.cpp), copy planner (plan.cpp) and host-side work-queue
// entry builders (rdmaxcel_host.cpp), meant to be
// built with -fsanitize=address,undefined: random valid and invalid Slices go through every host entry
// point, and what comes back is checked against the definitions (iter == get, index(get(i)) == i,
// the canonical form decodes to the same byte offsets as get).  No GPU, no HIP headers.
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../monarch_amd/csrc/mhip_internal.h"

using namespace mhip;

static uint64_t rng_state = 0x9e3779b97f4a7c15ull;
static uint64_t rnd() {
    rng_state ^= rng_state << 13;
    rng_state ^= rng_state >> 7;
    rng_state ^= rng_state << 17;
    return rng_state;
}
static uint64_t below(uint64_t n) { return rnd() % n; }

#define CHECK(cond)                                                                  \
    do {                                                                             \
        if (!(cond)) {                                                               \
            std::printf("FAILED %s at line %d (case %" PRIu64 ")\n", #cond, __LINE__, case_no); \
            std::exit(1);                                                            \
        }                                                                            \
    } while (0)

static uint64_t case_no = 0;

// byte offset of packed byte `byte` by the definition: element get(i), byte within the element
static uint64_t byte_by_definition(const mhip_slice_t& s, uint32_t elem_size, uint64_t byte) {
    uint64_t loc = 0;
    const int rc = mhip_slice_get(&s, byte / elem_size, &loc);
    if (rc != MHIP_SUCCESS) {
        std::printf("get failed with %d\n", rc);
        std::exit(1);
    }
    return loc * elem_size + byte % elem_size;
}

// the same through the canonical form: row-major decode of the dimensions outside the run
static uint64_t byte_by_canonical_form(const CanonSlice& c, uint32_t unit, uint64_t byte, uint64_t skew = 0) {
    const uint64_t t = byte / unit;
    uint64_t row = t / c.run, off = c.offset + t % c.run;
    for (int k = c.ndim - 1; k >= 0; --k) {
        off += (row % c.dims[k].size) * c.dims[k].stride;
        row /= c.dims[k].size;
    }
    return off * unit + byte % unit + skew;
}

int main() {
    const uint32_t elem_sizes[] = {1, 2, 3, 4, 6, 8, 12, 16};
    uint64_t n_valid = 0, n_invalid = 0;
    for (case_no = 0; case_no < 8000; ++case_no) {
        // a valid slice: row-major over a random permutation of the dimensions, with random gaps
        const uint32_t nd = (uint32_t)below(6);
        std::vector<uint64_t> sizes(nd), strides(nd);
        std::vector<uint32_t> order(nd);
        for (uint32_t k = 0; k < nd; ++k) {
            sizes[k] = 1 + below(7);
            order[k] = k;
        }
        for (uint32_t k = nd; k > 1; --k) std::swap(order[k - 1], order[below(k)]);
        uint64_t step = 1 + (below(4) == 0 ? below(3) : 0);
        for (uint32_t j = 0; j < nd; ++j) {
            const uint32_t k = order[j];
            strides[k] = step;
            step *= sizes[k] * (1 + (below(3) == 0 ? below(3) : 0));
        }
        bool mutated = false;  // set when a change may have made the slice invalid
        if (nd && below(10) == 0) {  // empty; invalid when the dimension shared its stride as one of size 1
            sizes[below(nd)] = 0;
            mutated = true;
        }
        if (nd && below(4) == 0) {
            strides[below(nd)] = below(2) ? below(40) : strides[below(nd)];
            mutated = true;
        }
        const uint64_t offset = below(50);
        mhip_slice_t s{offset, nd, sizes.data(), strides.data()};

        const int rc = mhip_slice_validate(offset, sizes.data(), nd, strides.data(), nd);
        CHECK(mutated || rc == MHIP_SUCCESS);
        if (rc != MHIP_SUCCESS) {
            ++n_invalid;
            CHECK(rc >= 10000);
            continue;
        }
        ++n_valid;
        uint64_t len = 0;
        CHECK(mhip_slice_len(&s, &len) == MHIP_SUCCESS);
        uint64_t expect_len = 1;
        for (uint64_t v : sizes) expect_len *= v;
        CHECK(len == expect_len);
        int contiguous = -1;
        CHECK(mhip_slice_is_contiguous(&s, &contiguous) == MHIP_SUCCESS);

        // iter == get, in pieces that start anywhere; index(get(i)) == i; bounds hold
        std::vector<uint64_t> locs(len + 3, ~0ull);
        uint64_t done = 0;
        while (done < len) {
            const uint64_t want = 1 + below(len);
            uint64_t written = 0;
            CHECK(mhip_slice_iter(&s, done, want, locs.data() + done, &written) == MHIP_SUCCESS);
            CHECK(written == (want < len - done ? want : len - done));
            done += written;
        }
        uint64_t written = 7;
        CHECK(mhip_slice_iter(&s, len, 5, locs.data() + len, &written) == MHIP_SUCCESS && written == 0);
        uint64_t lo = 0, hi = 0;
        const int brc = mhip_slice_bounds(&s, &lo, &hi);
        CHECK(len == 0 || brc == MHIP_SUCCESS);
        std::vector<uint64_t> coords(nd + 1);
        for (uint64_t i = 0; i < len; ++i) {
            uint64_t loc = 0, index = ~0ull;
            CHECK(mhip_slice_get(&s, i, &loc) == MHIP_SUCCESS && loc == locs[i]);
            CHECK(loc >= lo && loc <= hi);
            CHECK(mhip_slice_index(&s, loc, &index) == MHIP_SUCCESS && index == i);
            CHECK(mhip_slice_coordinates(&s, loc, coords.data()) == MHIP_SUCCESS);
            uint64_t back = 0;
            CHECK(mhip_slice_location(&s, coords.data(), nd, &back) == MHIP_SUCCESS && back == loc);
        }
        uint64_t loc = 0;
        CHECK(mhip_slice_get(&s, len, &loc) == MHIP_ERR_INDEX_OUT_OF_RANGE);
        if (contiguous == 1)
            for (uint64_t i = 0; i < len; ++i) CHECK(locs[i] == offset + i);

        // select / at produce slices whose elements are elements of s
        if (nd && len) {
            const uint32_t dim = (uint32_t)below(nd);
            std::vector<uint64_t> osz(nd), ost(nd);
            uint64_t ooff = 0;
            const uint64_t b = below(sizes[dim]), e = b + 1 + below(sizes[dim] - b), st = 1 + below(3);
            // a step can leave a stride that an outer stride is no multiple of, or that is too small for
            // the dimension sorted after it: the result is then refused, as Slice::select refuses it when
            // it re-validates (slice.rs:325)
            const int src = mhip_slice_select(&s, dim, b, e, st, &ooff, osz.data(), ost.data());
            CHECK(src == MHIP_SUCCESS || (st > 1 && (src == MHIP_ERR_NONRECTANGULAR_SHAPE || src == MHIP_ERR_STRIDE_TOO_SMALL)));
            if (src == MHIP_SUCCESS) {
                mhip_slice_t sub{ooff, nd, osz.data(), ost.data()};
                uint64_t sublen = 0;
                CHECK(mhip_slice_len(&sub, &sublen) == MHIP_SUCCESS && sublen >= 1 && sublen <= len);
                for (uint64_t i = 0; i < sublen; ++i) {
                    uint64_t l = 0, idx = 0;
                    CHECK(mhip_slice_get(&sub, i, &l) == MHIP_SUCCESS);
                    CHECK(mhip_slice_index(&s, l, &idx) == MHIP_SUCCESS);
                }
                CHECK(mhip_slice_enforce_embedding(&sub, &s) == MHIP_SUCCESS);
            }
            std::vector<uint64_t> asz(nd), ast(nd);
            uint64_t aoff = 0;
            CHECK(mhip_slice_at(&s, dim, b, &aoff, asz.data(), ast.data()) == MHIP_SUCCESS);
            CHECK(mhip_slice_at(&s, dim, sizes[dim], &aoff, asz.data(), ast.data()) != MHIP_SUCCESS);
        }

        // view: a reshape of the same element count succeeds exactly when the slice starts at 0 and every offset of
        // [0, len) is one of its locations (slice.rs:579-635); the strides that come back are row-major
        if (len && len <= 4096) {
            uint64_t ns[3] = {1, 1, 1};
            uint64_t rest = len;
            for (int k = 0; k < 2; ++k) {
                uint64_t f = 1 + below(rest < 9 ? rest : 9);
                while (rest % f) --f;
                ns[k] = f;
                rest /= f;
            }
            ns[2] = rest;
            uint64_t vst[3] = {7, 7, 7};
            const int vrc = mhip_slice_view(&s, ns, 3, vst);
            std::vector<char> member(len, 0);
            bool dense = offset == 0;
            for (uint64_t i = 0; i < len && dense; ++i) {
                if (locs[i] >= len) dense = false;
                else member[locs[i]] = 1;
            }
            for (uint64_t i = 0; i < len && dense; ++i) dense = member[i] != 0;
            CHECK((vrc == MHIP_SUCCESS) == dense);
            if (vrc == MHIP_SUCCESS) CHECK(vst[2] == 1 && vst[1] == ns[2] && vst[0] == ns[1] * ns[2]);
            else CHECK(vrc == MHIP_ERR_INCOMPATIBLE_VIEW);
            ns[2] += 1;
            CHECK(mhip_slice_view(&s, ns, 3, vst) == MHIP_ERR_INCOMPATIBLE_VIEW);   // another element count
            const uint64_t wrap[2] = {1ull << 32, 1ull << 32};                     // a product that wraps to 0
            CHECK(mhip_slice_view(&s, wrap, 2, vst) == MHIP_ERR_INCOMPATIBLE_VIEW);
        }

        // the planner: every packed byte lands where the definition says, for several element sizes,
        // address alignments and unit limits
        for (int rep = 0; rep < 3; ++rep) {
            const uint32_t es = elem_sizes[below(8)];
            const uint64_t mask = below(3) == 0 ? below(64) : 0;
            const uint32_t max_unit = 1u << below(5);
            CanonSlice c;
            uint32_t unit = 0;
            const bool nonempty = canonicalize(s, es, mask, max_unit, &c, &unit);
            CHECK(nonempty == (len != 0));
            if (!nonempty) continue;
            CHECK(unit >= 1 && unit <= max_unit && (unit & (unit - 1)) == 0 && (mask & (unit - 1)) == 0);
            CHECK(c.total * unit == len * es && c.run >= 1 && c.ndim >= 0 && c.ndim <= (int)nd + 1);
            CHECK(same_shape(c, c));
            uint64_t rows = 1;
            for (int k = 0; k < c.ndim; ++k) rows *= c.dims[k].size;
            CHECK(rows * c.run == c.total);
            const uint64_t nbytes = len * es;
            const uint64_t stride = nbytes > 4096 ? 1 + below(7) : 1;  // sample long ones
            for (uint64_t byte = below(stride); byte < nbytes; byte += stride)
                CHECK(byte_by_canonical_form(c, unit, byte) == byte_by_definition(s, es, byte));
            // the form whose unit the view's own offset does not limit: at least as coarse, same bytes
            CanonSlice r;
            uint32_t unit_r = 0;
            uint64_t skew = ~0ull;
            CHECK(canonicalize(s, es, mask, max_unit, &r, &unit_r, &skew));
            CHECK(unit_r >= unit && unit_r <= max_unit && (unit_r & (unit_r - 1)) == 0 && (mask & (unit_r - 1)) == 0);
            CHECK(skew < unit_r && r.total * unit_r == len * es && r.ndim == c.ndim);
            for (uint64_t byte = below(stride); byte < nbytes; byte += stride)
                CHECK(byte_by_canonical_form(r, unit_r, byte, skew) == byte_by_definition(s, es, byte));
        }

        // a mesh over the same slice: the members of each dimension contain the rank itself
        if (nd && len && len <= 512) {
            const uint64_t rank = locs[below(len)];
            for (uint32_t dim = 0; dim < nd; ++dim) {
                std::vector<uint64_t> members(sizes[dim] + 1, ~0ull);
                uint64_t dim_rank = ~0ull;
                CHECK(mhip_mesh_dim_members(&s, rank, dim, members.data(), &dim_rank) == MHIP_SUCCESS);
                CHECK(dim_rank < sizes[dim] && members[dim_rank] == rank && members[sizes[dim]] == ~0ull);
            }
            // the reduce group of a random list of dimensions, in the caller's order: row-major over those dimensions,
            // the rank's own coordinates everywhere else (device_mesh.rs:120-177)
            uint32_t dims[8];
            uint32_t ndims = (uint32_t)below(nd + 1);
            std::vector<uint32_t> pool(nd);
            for (uint32_t k = 0; k < nd; ++k) pool[k] = k;
            for (uint32_t k = nd; k > 1; --k) std::swap(pool[k - 1], pool[below(k)]);
            uint64_t group = 1;
            for (uint32_t d = 0; d < ndims; ++d) { dims[d] = pool[d]; group *= sizes[pool[d]]; }
            std::vector<uint64_t> out(group + 1, ~0ull);
            uint64_t count = ~0ull;
            CHECK(mhip_mesh_ranks_for_dims(&s, rank, dims, ndims, out.data(), group, &count) == MHIP_SUCCESS);
            if (ndims == 0) {
                CHECK(count == 0);
            } else {
                CHECK(count == group && out[group] == ~0ull);
                std::vector<uint64_t> own(nd), c(nd);
                CHECK(mhip_slice_coordinates(&s, rank, own.data()) == MHIP_SUCCESS);
                bool has_self = false;
                for (uint64_t i = 0; i < group; ++i) {
                    c = own;
                    uint64_t rem = i;
                    for (uint32_t d = ndims; d-- > 0;) { c[dims[d]] = rem % sizes[dims[d]]; rem /= sizes[dims[d]]; }
                    uint64_t want = 0;
                    CHECK(mhip_slice_location(&s, c.data(), nd, &want) == MHIP_SUCCESS);
                    CHECK(out[i] == want);
                    has_self |= out[i] == rank;
                }
                CHECK(has_self);
                if (group > 1) CHECK(mhip_mesh_ranks_for_dims(&s, rank, dims, ndims, out.data(), group - 1, &count) == MHIP_ERR_INVALID_ARGUMENT);
                dims[0] = nd;
                CHECK(mhip_mesh_ranks_for_dims(&s, rank, dims, ndims, out.data(), group, &count) == MHIP_ERR_DIMENSION_OUT_OF_RANGE);
            }
        }
    }
    // caller-built structs that Slice::new would never produce, and extreme arguments: a status comes back, nothing
    // divides by zero, wraps or reads out of bounds
    {
        case_no = 100000;
        uint64_t out[4] = {0, 0, 0, 0}, w = 99;
        const uint64_t four = 4, zero = 0, one = 1;
        const mhip_slice_t zero_stride{0, 1, &four, &zero};
        CHECK(mhip_slice_coordinates(&zero_stride, 2, out) == MHIP_ERR_INVALID_ARGUMENT);
        CHECK(mhip_slice_index(&zero_stride, 0, out) == MHIP_ERR_INVALID_ARGUMENT);
        CHECK(mhip_slice_enforce_embedding(&zero_stride, &zero_stride) == MHIP_ERR_INVALID_ARGUMENT);
        uint64_t members[4];
        CHECK(mhip_mesh_dim_members(&zero_stride, 0, 0, members, out) == MHIP_ERR_INVALID_ARGUMENT);
        const mhip_slice_t plain{0, 1, &four, &one};
        const uint64_t huge = ~0ull, two = 2;
        CHECK(mhip_slice_subview(&plain, &huge, 1, &two, 1, out) == MHIP_ERR_INDEX_OUT_OF_RANGE);   // starts + lens wraps to 1
        CHECK(mhip_slice_subview(&plain, &two, 1, &huge, 1, out) == MHIP_ERR_INDEX_OUT_OF_RANGE);
        CHECK(mhip_slice_subview(&plain, &two, 1, &two, 1, out) == MHIP_SUCCESS && out[0] == 2);
        uint64_t locs[4] = {7, 7, 7, 7};
        CHECK(mhip_slice_iter(&plain, 1, huge, locs, &w) == MHIP_SUCCESS && w == 3 && locs[0] == 1 && locs[2] == 3);  // start + count wraps
        CHECK(mhip_slice_iter(&plain, huge, huge, locs, &w) == MHIP_SUCCESS && w == 0);
        const mhip_slice_t too_deep{0, MHIP_MAX_DIMS + 1, &four, &one};
        CHECK(mhip_slice_len(&too_deep, out) == MHIP_ERR_INVALID_ARGUMENT);
        const mhip_slice_t null_arrays{0, 2, nullptr, nullptr};
        CHECK(mhip_slice_get(&null_arrays, 0, out) == MHIP_ERR_INVALID_ARGUMENT);
    }

    // SendTensor routing: the i-th sender pairs with the i-th receiver; to_mesh checks on random name lists
    for (case_no = 200000; case_no < 202000; ++case_no) {
        const uint64_t n_from = 1 + below(6), n_to = 1 + below(6), s_from = 1 + below(3), s_to = 1 + below(3);
        const uint64_t o_from = below(10), o_to = below(30);
        const mhip_slice_t from{o_from, 1, &n_from, &s_from}, to{o_to, 1, &n_to, &s_to};
        for (uint64_t rank = 0; rank < 50; ++rank) {
            uint64_t fr = 1, tr = 1;
            CHECK(mhip_send_tensor_route(&from, &to, rank, &fr, &tr) == MHIP_SUCCESS);
            uint64_t want_to = MHIP_NO_RANK, want_from = MHIP_NO_RANK;
            if (rank >= o_from && (rank - o_from) % s_from == 0 && (rank - o_from) / s_from < n_from) {
                const uint64_t i = (rank - o_from) / s_from;
                if (i < n_to) want_to = o_to + i * s_to;
            }
            if (rank >= o_to && (rank - o_to) % s_to == 0 && (rank - o_to) / s_to < n_to) {
                const uint64_t i = (rank - o_to) / s_to;
                if (i < n_from) want_from = o_from + i * s_from;
            }
            CHECK(fr == want_from && tr == want_to);
        }
        const char* pool[] = {"host", "gpu", "replica", "pp"};
        const uint32_t nm = (uint32_t)below(5), ns = (uint32_t)below(4);
        const char* mesh_names[4];
        const char* slicing_names[4];
        uint64_t mesh_sizes[4], sl_sizes[4], sl_strides[4];
        uint32_t perm[4] = {0, 1, 2, 3};
        for (uint32_t k = 4; k > 1; --k) std::swap(perm[k - 1], perm[below(k)]);
        for (uint32_t m = 0; m < nm; ++m) { mesh_names[m] = pool[perm[m]]; mesh_sizes[m] = 1 + below(3); }
        uint32_t perm2[4] = {0, 1, 2, 3};
        for (uint32_t k = 4; k > 1; --k) std::swap(perm2[k - 1], perm2[below(k)]);
        for (uint32_t k = 0; k < ns; ++k) { slicing_names[k] = pool[perm2[k]]; sl_sizes[k] = 1 + below(3); sl_strides[k] = 1 + below(9); }
        const mhip_slice_t slicing{below(5), ns, sl_sizes, sl_strides};
        uint64_t osz[4], ost[4];
        uint32_t ond = 77, bc[4], nbc = 77, culprit = 77;
        const int rc = mhip_to_mesh_from_ranks(slicing_names, &slicing, mesh_names, mesh_sizes, nm, osz, ost, &ond, bc, &nbc, &culprit);
        // by the definition (tensor.py:417-437)
        int want = MHIP_SUCCESS;
        uint32_t kept = 0, nb = 0;
        for (uint32_t m = 0; m < nm && want == MHIP_SUCCESS; ++m) {
            uint32_t idx = ns;
            for (uint32_t k = 0; k < ns; ++k) if (slicing_names[k] == mesh_names[m]) idx = k;   // pool strings are unique objects
            if (idx == ns) { ++nb; continue; }
            if (sl_sizes[idx] != mesh_sizes[m]) { want = MHIP_ERR_MESH_DIM_LENGTH_MISMATCH; break; }
            CHECK(rc != MHIP_SUCCESS || (osz[kept] == mesh_sizes[m] && ost[kept] == sl_strides[idx]));
            ++kept;
        }
        if (want == MHIP_SUCCESS && kept != ns) want = MHIP_ERR_MESH_DIM_MISSING;
        CHECK(rc == want);
        if (rc == MHIP_SUCCESS) CHECK(ond == kept && nbc == nb);
    }

    // Work-queue and completion-queue entries built on the calling thread (rdmaxcel_host.cpp).  Queues are heap blocks
    // of exactly the size the parameters describe, so a store outside a slot is an AddressSanitizer report; the bytes are
    // compared with the wire format written out one byte at a time (rdmaxcel-sys/src/rdmaxcel.cu:139-160,201-245,292-326).
    uint64_t n_entries = 0, n_refused = 0;
    for (int round = 0; round < 20000; ++round) {
        case_no = 2000000 + round;
        const uint32_t cnt = below(8) == 0 ? (uint32_t)below(70) : 1u << below(7);   // mostly powers of two, some not
        const bool pow2 = cnt != 0 && (cnt & (cnt - 1)) == 0;
        const size_t slots = cnt ? cnt : 1;
        uint8_t* sq = static_cast<uint8_t*>(std::aligned_alloc(64, slots * 64));
        uint32_t* dbrec = static_cast<uint32_t*>(std::aligned_alloc(8, 8));
        for (size_t i = 0; i < slots * 64; ++i) sq[i] = 0xA5;
        dbrec[0] = dbrec[1] = 0xDEADBEEFu;
        mhip_wqe_params_t p{};
        p.laddr = rnd();
        p.lkey = (uint32_t)rnd();
        p.wr_id = below(4) == 0 ? rnd() : below(4 * slots + 1);
        p.signaled = (uint8_t)below(2);
        p.op_type = below(3) == 0 ? MHIP_MLX5_OPCODE_RDMA_READ : below(2) ? MHIP_MLX5_OPCODE_RDMA_WRITE : MHIP_MLX5_OPCODE_RDMA_WRITE_IMM;
        p.raddr = rnd();
        p.rkey = (uint32_t)rnd();
        p.qp_num = (uint32_t)below(1u << 24);
        p.length = below(3) == 0 ? rnd() : below(1u << 20);
        p.buf = sq;
        p.dbrec = dbrec;
        p.wqe_cnt = cnt;
        const unsigned spoil = (unsigned)below(12);     // 0..3 spoil one argument
        if (spoil == 0) p.buf = nullptr;
        if (spoil == 1) p.dbrec = nullptr;
        if (spoil == 2) p.buf = sq + 4 * (1 + below(3));
        if (spoil == 3) p.dbrec = reinterpret_cast<uint32_t*>(reinterpret_cast<uint8_t*>(dbrec) + 1 + below(3));
        const bool bad = spoil < 4 || !pow2;
        int rc = mhip_rdmaxcel_send_wqe_host(&p);
        CHECK((rc == MHIP_SUCCESS) == !bad);
        if (rc != MHIP_SUCCESS) {
            CHECK(rc == MHIP_ERR_INVALID_ARGUMENT);
            for (size_t i = 0; i < slots * 64; ++i) CHECK(sq[i] == 0xA5);
            CHECK(dbrec[0] == 0xDEADBEEFu && dbrec[1] == 0xDEADBEEFu);
            ++n_refused;
        } else {
            const uint32_t idx = (uint32_t)p.wr_id;
            const size_t at = (size_t)(idx & (cnt - 1)) * 64;
            uint8_t want[48] = {0};
            const uint32_t w0 = (idx << 8) | p.op_type, w1 = (p.qp_num << 8) | 3u, len = (uint32_t)p.length;
            for (int b = 0; b < 4; ++b) { want[b] = (uint8_t)(w0 >> (24 - 8 * b)); want[4 + b] = (uint8_t)(w1 >> (24 - 8 * b)); }
            want[11] = p.signaled ? 0x0A : 0x00;
            for (int b = 0; b < 8; ++b) { want[16 + b] = (uint8_t)(p.raddr >> (56 - 8 * b)); want[40 + b] = (uint8_t)(p.laddr >> (56 - 8 * b)); }
            for (int b = 0; b < 4; ++b) { want[24 + b] = (uint8_t)(p.rkey >> (24 - 8 * b)); want[32 + b] = (uint8_t)(len >> (24 - 8 * b)); want[36 + b] = (uint8_t)(p.lkey >> (24 - 8 * b)); }
            for (size_t i = 0; i < slots * 64; ++i) CHECK(sq[i] == (i >= at && i < at + 48 ? want[i - at] : 0xA5));
            const uint32_t rec = (idx + 1u) & 0xFFFFFFu;
            const uint8_t* d = reinterpret_cast<const uint8_t*>(dbrec + 1);
            CHECK(d[0] == 0 && d[1] == (uint8_t)(rec >> 16) && d[2] == (uint8_t)(rec >> 8) && d[3] == (uint8_t)rec);
            CHECK(dbrec[0] == 0xDEADBEEFu);
            ++n_entries;
        }

        // the receive entry: 16 bytes at buf itself, any wqe_cnt
        uint8_t* rq = static_cast<uint8_t*>(std::aligned_alloc(16, 16));
        for (int i = 0; i < 16; ++i) rq[i] = 0x5A;
        dbrec[0] = dbrec[1] = 0xDEADBEEFu;
        p.buf = spoil == 0 ? nullptr : spoil == 2 ? rq + 8 : rq;
        rc = mhip_rdmaxcel_recv_wqe_host(&p);
        CHECK((rc == MHIP_SUCCESS) == (spoil >= 4));
        if (rc == MHIP_SUCCESS) {
            const uint32_t len = (uint32_t)p.length, rec = (uint32_t)(p.wr_id + 1);
            for (int b = 0; b < 4; ++b) CHECK(rq[b] == (uint8_t)(len >> (24 - 8 * b)) && rq[4 + b] == (uint8_t)(p.lkey >> (24 - 8 * b)));
            for (int b = 0; b < 8; ++b) CHECK(rq[8 + b] == (uint8_t)(p.laddr >> (56 - 8 * b)));
            const uint8_t* d = reinterpret_cast<const uint8_t*>(dbrec);
            for (int b = 0; b < 4; ++b) CHECK(d[b] == (uint8_t)(rec >> (24 - 8 * b)));
            CHECK(dbrec[1] == 0xDEADBEEFu);
            ++n_entries;
        } else {
            for (int i = 0; i < 16; ++i) CHECK(rq[i] == 0x5A);
            ++n_refused;
        }

        // the doorbell ring: exactly 64 bytes, 8-byte aligned both sides
        uint8_t* reg = static_cast<uint8_t*>(std::aligned_alloc(8, 64));
        for (int i = 0; i < 64; ++i) reg[i] = 0;
        const size_t from = (size_t)below(slots) * 64;
        const unsigned skew = below(6) == 0 ? 1 + (unsigned)below(7) : 0;
        rc = mhip_rdmaxcel_db_ring_host(skew && below(2) ? static_cast<void*>(reg + skew) : static_cast<void*>(reg),
                                        skew ? static_cast<const void*>(sq + from + skew) : static_cast<const void*>(sq + from));
        CHECK((rc == MHIP_SUCCESS) == (skew == 0));
        if (rc == MHIP_SUCCESS) for (int i = 0; i < 64; ++i) CHECK(reg[i] == sq[from + i]);
        else for (int i = 0; i < 64; ++i) CHECK(reg[i] == 0);
        CHECK(mhip_rdmaxcel_db_ring_host(nullptr, sq) == MHIP_ERR_INVALID_ARGUMENT);
        std::free(reg);
        std::free(rq);

        // one look at a completion queue of cqe_cnt entries of 64 or 128 bytes
        const uint32_t csize = below(10) == 0 ? (uint32_t)(4 * below(40)) : below(2) ? 64u : 128u;
        const bool cq_ok = pow2 && (csize == 64 || csize == 128);
        const size_t cq_bytes = slots * (csize ? csize : 4);
        uint8_t* cq = static_cast<uint8_t*>(std::aligned_alloc(64, (cq_bytes + 63) / 64 * 64));
        for (size_t i = 0; i < cq_bytes; ++i) cq[i] = (uint8_t)rnd();
        mhip_cqe_poll_params_t q{};
        q.cqe_buf = cq;
        q.cqe_size = csize;
        q.consumer_index = below(3) == 0 ? (uint32_t)rnd() : (uint32_t)below(4 * slots + 1);
        q.cqe_cnt = cnt;
        q.dbrec = dbrec;
        dbrec[0] = dbrec[1] = 0xDEADBEEFu;
        int32_t result = -1;
        rc = mhip_rdmaxcel_cqe_poll_host(&result, &q);
        CHECK((rc == MHIP_SUCCESS) == cq_ok);
        if (rc == MHIP_SUCCESS) {
            const uint8_t* e = cq + (size_t)(q.consumer_index & (cnt - 1)) * csize;
            const uint8_t op_own = e[csize - 1];
            const bool owned = (uint32_t)(op_own & 1) == ((q.consumer_index / cnt) & 1u) && (op_own >> 4) != 0xF;
            if (!owned) {
                CHECK(result == -1 && dbrec[0] == 0xDEADBEEFu);
            } else {
                const uint32_t bc = (uint32_t)e[44] << 24 | (uint32_t)e[45] << 16 | (uint32_t)e[46] << 8 | e[47];
                CHECK(result == ((op_own >> 4) < 4 ? (int32_t)bc : -2));
                const uint32_t rec = (q.consumer_index + 1u) & 0xFFFFFFu;
                const uint8_t* d = reinterpret_cast<const uint8_t*>(dbrec);
                CHECK(d[0] == 0 && d[1] == (uint8_t)(rec >> 16) && d[2] == (uint8_t)(rec >> 8) && d[3] == (uint8_t)rec);
            }
            CHECK(dbrec[1] == 0xDEADBEEFu);
            ++n_entries;
        } else {
            CHECK(rc == MHIP_ERR_INVALID_ARGUMENT && result == -1 && dbrec[0] == 0xDEADBEEFu);
            ++n_refused;
        }
        CHECK(mhip_rdmaxcel_cqe_poll_host(nullptr, &q) == MHIP_ERR_INVALID_ARGUMENT);
        std::free(cq);
        std::free(dbrec);
        std::free(sq);
    }
    CHECK(n_entries > 20000 && n_refused > 2000);
    std::printf("ok: %" PRIu64 " queue entries built and %" PRIu64 " calls refused\n", n_entries, n_refused);

    std::printf("ok: %" PRIu64 " valid and %" PRIu64 " invalid slices\n", n_valid, n_invalid);
    return 0;
}
