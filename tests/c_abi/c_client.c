/* A plain-C client of include/monarch_hip.h: the shape of the call sequence a host-language
 * binding makes (device memory and streams through the runtime pass-through, then the data
 * path), with nothing but libc around it.  It checks results against loops written here, so
 * it depends neither on Python nor on the test oracle.  Exit code 0 and "c_client ok" on success.
 *
 *   gcc -std=c11 -O1 -I include tests/c_abi/c_client.c -o tests/c_abi/c_client \
 *       -L monarch_amd -lmonarch_hip -Wl,-rpath,'$ORIGIN/../../monarch_amd' -lm
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "monarch_hip.h"

#define CHECK(call)                                                                      \
    do {                                                                                 \
        int rc_ = (call);                                                                \
        if (rc_ != MHIP_SUCCESS) {                                                       \
            fprintf(stderr, "%s:%d: %s -> %d (%s)\n", __FILE__, __LINE__, #call, rc_,    \
                    mhip_error_string(rc_));                                             \
            return 1;                                                                    \
        }                                                                                \
    } while (0)

static uint32_t lcg(uint32_t* s) { return *s = *s * 1664525u + 1013904223u; }

static uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
static float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

int main(void) {
    int ndev = 0;
    CHECK(mhip_device_count(&ndev));
    if (ndev < 1) {
        fprintf(stderr, "no device\n");
        return 2;
    }
    CHECK(mhip_set_device(0));
    mhip_stream_t stream = NULL;
    CHECK(mhip_stream_create(&stream));

    /* 1. every other row of a [4,256,256] f32 tensor, packed and unpacked (configuration 1) */
    enum { N = 4 * 256 * 256, P = 4 * 128 * 256 };
    float* x = malloc(N * sizeof(float));
    float* packed = malloc(P * sizeof(float));
    float* back = malloc(N * sizeof(float));
    uint32_t seed = 1;
    for (int i = 0; i < N; ++i) x[i] = (float)(lcg(&seed) >> 8) / 8388608.0f - 1.0f;
    void *dx, *dp, *db;
    CHECK(mhip_malloc(&dx, N * sizeof(float)));
    CHECK(mhip_malloc(&dp, P * sizeof(float)));
    CHECK(mhip_malloc(&db, N * sizeof(float)));
    CHECK(mhip_memcpy_htod(dx, x, N * sizeof(float), stream));
    CHECK(mhip_memset(db, 0, N * sizeof(float), stream));
    const uint64_t sizes[3] = {4, 128, 256}, strides[3] = {65536, 512, 1};
    CHECK(mhip_slice_validate(0, sizes, 3, strides, 3));
    const mhip_slice_t view = {0, 3, sizes, strides};
    CHECK(mhip_slice_pack(dp, dx, &view, sizeof(float), stream));
    CHECK(mhip_slice_unpack(db, dp, &view, sizeof(float), stream));
    CHECK(mhip_memcpy_dtoh(packed, dp, P * sizeof(float), stream));
    CHECK(mhip_memcpy_dtoh(back, db, N * sizeof(float), stream));
    CHECK(mhip_stream_synchronize(stream));
    for (int a = 0, i = 0; a < 4; ++a)
        for (int r = 0; r < 128; ++r)
            for (int c = 0; c < 256; ++c, ++i) {
                const float want = x[a * 65536 + r * 512 + c];
                if (packed[i] != want || back[a * 65536 + r * 512 + c] != want) {
                    fprintf(stderr, "pack/unpack mismatch at %d\n", i);
                    return 1;
                }
            }
    for (int a = 0; a < 4; ++a)
        for (int r = 1; r < 256; r += 2)
            for (int c = 0; c < 256; ++c)
                if (back[a * 65536 + r * 256 + c] != 0.0f) {
                    fprintf(stderr, "unpack touched an element outside the view\n");
                    return 1;
                }

    /* 2. average of 8 bf16 buffers, fp32 accumulation in member order, one rounding */
    enum { M = 100003, G = 8 };
    uint16_t* h[G];
    void* d[G];
    const void* dptr[G];
    for (int g = 0; g < G; ++g) {
        h[g] = malloc(M * sizeof(uint16_t));
        for (int i = 0; i < M; ++i) h[g][i] = f32_to_bf16(((float)(lcg(&seed) >> 8) / 8388608.0f - 1.0f) * 0.02f);
        CHECK(mhip_malloc(&d[g], M * sizeof(uint16_t)));
        CHECK(mhip_memcpy_htod(d[g], h[g], M * sizeof(uint16_t), stream));
        dptr[g] = d[g];
    }
    void* dout;
    CHECK(mhip_malloc(&dout, M * sizeof(uint16_t)));
    mhip_event_t e0, e1;
    CHECK(mhip_event_create(&e0));
    CHECK(mhip_event_create(&e1));
    CHECK(mhip_event_record(e0, stream));
    CHECK(mhip_reduce(dout, dptr, G, M, MHIP_DTYPE_BF16, MHIP_OP_AVG, stream));
    CHECK(mhip_event_record(e1, stream));
    uint16_t* out = malloc(M * sizeof(uint16_t));
    CHECK(mhip_memcpy_dtoh(out, dout, M * sizeof(uint16_t), stream));
    CHECK(mhip_event_synchronize(e1));
    float ms = -1.0f;
    CHECK(mhip_event_elapsed_ms(&ms, e0, e1));
    CHECK(mhip_stream_synchronize(stream));
    for (int i = 0; i < M; ++i) {
        volatile float acc = bf16_to_f32(h[0][i]);
        for (int g = 1; g < G; ++g) acc = acc + bf16_to_f32(h[g][i]);
        acc = acc / 8.0f;
        if (out[i] != f32_to_bf16(acc)) {
            fprintf(stderr, "reduce mismatch at %d: %04x vs %04x\n", i, out[i], f32_to_bf16(acc));
            return 1;
        }
    }
    if (!(ms >= 0.0f)) {
        fprintf(stderr, "event timing failed\n");
        return 1;
    }

    /* 3. refusals come back as status codes, not as aborts */
    if (mhip_reduce(dout, dptr, G, M, MHIP_DTYPE_F8E4M3FN, MHIP_OP_SUM, stream) != MHIP_ERR_FLOAT8_REDUCTION) {
        fprintf(stderr, "an fp8 reduce was not refused\n");
        return 1;
    }
    const uint64_t bad_strides[3] = {65536, 128, 1};  /* rows of 256 elements only 128 apart: they overlap */
    if (mhip_slice_validate(0, sizes, 3, bad_strides, 3) != MHIP_ERR_STRIDE_TOO_SMALL) {
        fprintf(stderr, "overlapping rows were not refused\n");
        return 1;
    }

    /* 4. fp8 round trip: block maxima come back exactly (they encode to +-448) */
    enum { T = 5000 };
    uint16_t* t16 = malloc(T * sizeof(uint16_t));
    for (int i = 0; i < T; ++i) t16[i] = f32_to_bf16((float)(lcg(&seed) >> 8) / 8388608.0f - 1.0f);
    void *dt, *dq, *dsc, *dacc;
    const int nblk = (T + 1023) / 1024;
    CHECK(mhip_malloc(&dt, T * 2));
    CHECK(mhip_malloc(&dq, T));
    CHECK(mhip_malloc(&dsc, nblk * sizeof(float)));
    CHECK(mhip_malloc(&dacc, T * sizeof(float)));
    CHECK(mhip_memcpy_htod(dt, t16, T * 2, stream));
    CHECK(mhip_memset(dacc, 0, T * sizeof(float), stream));
    CHECK(mhip_fp8_quantize(dq, dsc, dt, T, 1024, stream));
    CHECK(mhip_fp8_dequant_accumulate(dacc, dq, dsc, T, 1024, stream));
    float* acc = malloc(T * sizeof(float));
    float* sc = malloc(nblk * sizeof(float));
    CHECK(mhip_memcpy_dtoh(acc, dacc, T * sizeof(float), stream));
    CHECK(mhip_memcpy_dtoh(sc, dsc, nblk * sizeof(float), stream));
    CHECK(mhip_stream_synchronize(stream));
    for (int b = 0; b < nblk; ++b) {
        float amax = 0.0f;
        int at = -1;
        for (int i = b * 1024; i < T && i < (b + 1) * 1024; ++i)
            if (fabsf(bf16_to_f32(t16[i])) > amax) {
                amax = fabsf(bf16_to_f32(t16[i]));
                at = i;
            }
        if (sc[b] != amax / 448.0f) {
            fprintf(stderr, "scale of block %d: %g vs %g\n", b, sc[b], amax / 448.0f);
            return 1;
        }
        /* float(448) * (amax / 448) is amax again up to one rounding of the product */
        if (fabsf(fabsf(acc[at]) - amax) > amax * 1.2e-7f) {
            fprintf(stderr, "block maximum of block %d not recovered: %g vs %g\n", b, acc[at], amax);
            return 1;
        }
        for (int i = b * 1024; i < T && i < (b + 1) * 1024; ++i)
            if (fabsf(acc[i] - bf16_to_f32(t16[i])) > sc[b] * 16.0f + 1e-30f) { /* half of the widest code spacing (32) */
                fprintf(stderr, "fp8 error too large at %d\n", i);
                return 1;
            }
    }

    /* 5. RdmaBuffer transfers in several work requests, max of the 8 buffers, stack, and a column block sent
     *    through staging memory (SendTensor) */
    {
        mhip_rdma_buffer_t local = {d[0], M * sizeof(uint16_t)}, remote = {dout, M * sizeof(uint16_t)};
        CHECK(mhip_buffer_read_into(&local, &remote, stream));            /* d[0] -> dout */
        uint32_t posted = 0;
        CHECK(mhip_buffer_transfer(d[1], dout, M * sizeof(uint16_t), 4096, stream, &posted)); /* dout -> d[1] */
        CHECK(mhip_memcpy_dtoh(out, d[1], M * sizeof(uint16_t), stream));
        CHECK(mhip_stream_synchronize(stream));
        if (posted != (M * sizeof(uint16_t) + 4095) / 4096 || memcmp(out, h[0], M * sizeof(uint16_t)) != 0) {
            fprintf(stderr, "segmented buffer transfer failed (%u requests)\n", posted);
            return 1;
        }
        memcpy(h[1], h[0], M * sizeof(uint16_t));
        mhip_rdma_buffer_t small = {dq, 16};
        if (mhip_buffer_read_into(&local, &small, stream) != MHIP_ERR_BUFFER_TOO_SMALL) {
            fprintf(stderr, "a write past the remote buffer was not refused\n");
            return 1;
        }
        CHECK(mhip_reduce(dout, dptr, G, M, MHIP_DTYPE_BF16, MHIP_OP_MAX, stream));
        CHECK(mhip_memcpy_dtoh(out, dout, M * sizeof(uint16_t), stream));
        CHECK(mhip_stream_synchronize(stream));
        for (int i = 0; i < M; ++i) {
            float best = bf16_to_f32(h[0][i]);
            for (int g = 1; g < G; ++g) best = bf16_to_f32(h[g][i]) > best ? bf16_to_f32(h[g][i]) : best;
            if (bf16_to_f32(out[i]) != best) {
                fprintf(stderr, "max mismatch at %d\n", i);
                return 1;
            }
        }
        void* dstack;
        CHECK(mhip_malloc(&dstack, (size_t)G * M * sizeof(uint16_t)));
        CHECK(mhip_stack(dstack, dptr, G, M, sizeof(uint16_t), stream));
        uint16_t* stacked = malloc((size_t)G * M * sizeof(uint16_t));
        CHECK(mhip_memcpy_dtoh(stacked, dstack, (size_t)G * M * sizeof(uint16_t), stream));
        CHECK(mhip_stream_synchronize(stream));
        for (int g = 0; g < G; ++g)
            if (memcmp(stacked + (size_t)g * M, h[g], M * sizeof(uint16_t)) != 0) {
                fprintf(stderr, "stack mismatch in member %d\n", g);
                return 1;
            }
        /* the eight members back out of the stack in one launch: 8 transfers of ragged length */
        {
            void* back[G];
            const void* from[G];
            size_t len[G];
            for (int g = 0; g < G; ++g) {
                CHECK(mhip_malloc(&back[g], M * sizeof(uint16_t)));
                CHECK(mhip_memset(back[g], 0, M * sizeof(uint16_t), stream));
                from[g] = (const char*)dstack + (size_t)g * M * sizeof(uint16_t);
                len[g] = M * sizeof(uint16_t) - 3 * (size_t)g;
            }
            uint32_t posted = 0;
            CHECK(mhip_buffer_transfer_many(back, from, len, G, 0, stream, &posted));
            for (int g = 0; g < G; ++g) {
                CHECK(mhip_memcpy_dtoh(out, back[g], M * sizeof(uint16_t), stream));
                CHECK(mhip_stream_synchronize(stream));
                const unsigned char* o = (const unsigned char*)out;
                int tail_ok = 1;  /* the 3 g bytes after a buffer's length keep their zeros */
                for (size_t i = len[g]; i < M * sizeof(uint16_t); ++i) tail_ok = tail_ok && o[i] == 0;
                if (posted != G || memcmp(o, h[g], len[g]) != 0 || !tail_ok) {
                    fprintf(stderr, "transfer of many buffers failed at buffer %d (%u requests)\n", g, posted);
                    return 1;
                }
                CHECK(mhip_free(back[g]));
            }
        }
        /* columns [64, 192) of the [1024, 256] f32 matrix at the start of x, sent as a [1024, 128] tensor */
        const uint64_t csizes[2] = {1024, 128}, cstrides[2] = {256, 1};
        const mhip_slice_t col = {64, 2, csizes, cstrides};
        uint64_t from_rank = 0, to_rank = 0;
        const uint64_t one = 1;
        const mhip_slice_t from_ranks = {0, 1, &one, &one}, to_ranks = {1, 1, &one, &one};
        CHECK(mhip_send_tensor_route(&from_ranks, &to_ranks, 1, &from_rank, &to_rank));
        if (from_rank != 0 || to_rank != MHIP_NO_RANK) {
            fprintf(stderr, "send_tensor routing: from %llu to %llu\n", (unsigned long long)from_rank, (unsigned long long)to_rank);
            return 1;
        }
        CHECK(mhip_send_tensor(db, 1024 * 128 * sizeof(float), dx, &col, sizeof(float), dp, stream));
        CHECK(mhip_memcpy_dtoh(back, db, 1024 * 128 * sizeof(float), stream));
        CHECK(mhip_stream_synchronize(stream));
        for (int r = 0; r < 1024; ++r)
            for (int c = 0; c < 128; ++c)
                if (back[r * 128 + c] != x[r * 256 + 64 + c]) {
                    fprintf(stderr, "send_tensor mismatch at row %d column %d\n", r, c);
                    return 1;
                }
        CHECK(mhip_free(dstack));
        free(stacked);
    }

    /* 6. device-initiated RDMA: a send WQE, the doorbell ring and one completion-queue poll on ordinary device
     * memory, against bytes written out by hand (mlx5 layouts: control, remote-address and data segment) */
    {
        enum { CNT = 4 };
        void *dsq, *ddb, *dreg, *dcq, *dres;
        CHECK(mhip_malloc(&dsq, CNT * 64)); CHECK(mhip_malloc(&ddb, 8)); CHECK(mhip_malloc(&dreg, 64));
        CHECK(mhip_malloc(&dcq, CNT * 64)); CHECK(mhip_malloc(&dres, 4));
        CHECK(mhip_memset(dsq, 0xEE, CNT * 64, stream)); CHECK(mhip_memset(ddb, 0, 8, stream));
        CHECK(mhip_memset(dcq, 0, CNT * 64, stream)); CHECK(mhip_memset(dres, 0xFF, 4, stream));   /* -1 */
        mhip_wqe_params_t w;
        memset(&w, 0, sizeof w);
        w.laddr = 0x00007F1234567890ull; w.lkey = 0xAABBCCDDu; w.length = 0x00100000; w.wr_id = 5; w.signaled = 1;
        w.op_type = MHIP_MLX5_OPCODE_RDMA_WRITE; w.raddr = 0x00007E00DEADBEE0ull; w.rkey = 0x11223344u; w.qp_num = 0x001234;
        w.buf = dsq; w.dbrec = ddb; w.wqe_cnt = CNT;
        CHECK(mhip_rdmaxcel_send_wqe(&w, stream));
        CHECK(mhip_rdmaxcel_ring_doorbells(dreg, dsq, 64, CNT, 5, 1, stream));
        /* the NIC's completion for consumer index 5: entry 1, second lap (owner bit 1), opcode 0, 1 MiB */
        unsigned char cqe[64];
        memset(cqe, 0, sizeof cqe);
        cqe[44] = 0x00; cqe[45] = 0x10; cqe[46] = 0x00; cqe[47] = 0x00; cqe[63] = 0x01;
        CHECK(mhip_memcpy_htod((char*)dcq + 64, cqe, 64, stream));
        mhip_cqe_poll_params_t c;
        c.cqe_buf = dcq; c.cqe_size = 64; c.consumer_index = 5; c.cqe_cnt = CNT; c.dbrec = (uint32_t*)ddb;
        CHECK(mhip_rdmaxcel_cqe_poll(dres, &c, stream));
        unsigned char sq[CNT * 64], reg[64], db[8];
        int32_t res = 0;
        CHECK(mhip_memcpy_dtoh(sq, dsq, sizeof sq, stream)); CHECK(mhip_memcpy_dtoh(reg, dreg, 64, stream));
        CHECK(mhip_memcpy_dtoh(db, ddb, 8, stream)); CHECK(mhip_memcpy_dtoh(&res, dres, 4, stream));
        CHECK(mhip_stream_synchronize(stream));
        static const unsigned char want[48] = {
            0x00, 0x00, 0x05, 0x08, 0x00, 0x12, 0x34, 0x03, 0x00, 0x00, 0x00, 0x0A, 0x00, 0x00, 0x00, 0x00,
            0x00, 0x00, 0x7E, 0x00, 0xDE, 0xAD, 0xBE, 0xE0, 0x11, 0x22, 0x33, 0x44, 0x00, 0x00, 0x00, 0x00,
            0x00, 0x10, 0x00, 0x00, 0xAA, 0xBB, 0xCC, 0xDD, 0x00, 0x00, 0x7F, 0x12, 0x34, 0x56, 0x78, 0x90};
        static const unsigned char want_db[8] = {0, 0, 0, 6, 0, 0, 0, 6};   /* CQ consumer 6 | send counter 6 */
        int ok = memcmp(sq + 64, want, 48) == 0 && memcmp(reg, sq + 64, 64) == 0 && memcmp(db, want_db, 8) == 0 && res == 0x00100000;
        for (int i = 0; i < CNT * 64; ++i)
            if ((i < 64 || i >= 112) && sq[i] != 0xEE) ok = 0;
        if (!ok) {
            fprintf(stderr, "rdmaxcel: WQE / doorbell / poll bytes differ (poll result %d)\n", (int)res);
            return 1;
        }
        /* the same WQE through the host function, into host memory */
        _Alignas(64) unsigned char hsq[CNT * 64];
        uint32_t hdb[2] = {0, 0};
        w.buf = hsq; w.dbrec = hdb;
        CHECK(mhip_rdmaxcel_send_wqe_host(&w));
        if (memcmp(hsq + 64, want, 48) != 0 || memcmp(&hdb[1], want_db + 4, 4) != 0) {
            fprintf(stderr, "rdmaxcel: host WQE bytes differ\n");
            return 1;
        }
        CHECK(mhip_free(dsq)); CHECK(mhip_free(ddb)); CHECK(mhip_free(dreg)); CHECK(mhip_free(dcq)); CHECK(mhip_free(dres));
    }

    for (int g = 0; g < G; ++g) CHECK(mhip_free(d[g]));
    CHECK(mhip_free(dx)); CHECK(mhip_free(dp)); CHECK(mhip_free(db)); CHECK(mhip_free(dout));
    CHECK(mhip_free(dt)); CHECK(mhip_free(dq)); CHECK(mhip_free(dsc)); CHECK(mhip_free(dacc));
    CHECK(mhip_event_destroy(e0)); CHECK(mhip_event_destroy(e1));
    CHECK(mhip_stream_destroy(stream));
    printf("c_client ok (reduce of 8 x %d bf16: %.3f ms)\n", (int)M, ms);
    return 0;
}
