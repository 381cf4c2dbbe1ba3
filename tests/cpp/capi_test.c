/* The kernel-level C ABI used from plain C, with nothing but the library itself: device memory
 * from cx_device_alloc, host <-> device copies with cx_copy.  One error-feedback step (whole-vector
 * top-k threshold, fused compress), the receive side (decompress, add), the run-length codec,
 * and the status codes of the error paths.  Prints the PASSED / FAILED line of the other tests. */
#include <comprex_gfx950.h>

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static int errors = 0;
#define CHECK(cond)                                                         \
    do {                                                                    \
        if (!(cond)) {                                                      \
            printf("line %d: %s  [%s]\n", __LINE__, #cond, cx_last_error()); \
            ++errors;                                                       \
        }                                                                   \
    } while (0)

int main(void) {
    if (cx_device_count() < 1) {
        printf("no GPU: this test drives the HIP library and cannot run here\n");
        return 77;
    }
    enum { N = 100000 };
    const float topK = 0.01f;
    float* g = malloc(N * sizeof(float));
    float* r = malloc(N * sizeof(float));
    float* back = malloc(N * sizeof(float));
    unsigned x = 7u;
    for (int i = 0; i < N; ++i) {
        x = x * 1664525u + 1013904223u;
        g[i] = (float)((int)((x >> 8) % 20001u) - 10000) / 16.0f;
        r[i] = (float)(i % 13) / 4.0f;
    }
    cx_handle h = NULL;
    CHECK(cx_create(&h, NULL) == CX_OK);
    void *d_g = NULL, *d_r = NULL, *d_msg = NULL, *d_dense = NULL, *d_rle = NULL;
    const long long cap = 8 + 8ll * N, rle_cap = 16 + 4ll * N + 4ll * (N + 1);
    CHECK(cx_device_alloc(&d_g, N * sizeof(float)) == CX_OK);
    CHECK(cx_device_alloc(&d_r, N * sizeof(float)) == CX_OK);
    CHECK(cx_device_alloc(&d_dense, N * sizeof(float)) == CX_OK);
    CHECK(cx_device_alloc(&d_msg, (size_t)cap) == CX_OK);
    CHECK(cx_device_alloc(&d_rle, (size_t)rle_cap) == CX_OK);
    CHECK(cx_pointer_on_device(d_g) == 1 && cx_pointer_on_device(g) == 0);
    CHECK(cx_copy(h, d_g, g, N * sizeof(float)) == CX_OK);
    CHECK(cx_copy(h, d_r, r, N * sizeof(float)) == CX_OK);

    /* threshold = the (pos+1)-th largest |r + g| of the whole vector (more sub-samples than elements) */
    float thr = -1.0f;
    CHECK(cx_topk_threshold(h, CX_F32, d_r, d_g, N, N, topK, 1 << 20, 10.0f, NULL, &thr) == CX_OK);
    const int pos = cx_topk_pos(N, topK);
    int greater = 0, equal = 0;
    for (int i = 0; i < N; ++i) {
        const float s = fabsf(r[i] + g[i]);
        greater += s > thr;
        equal += s == thr;
    }
    CHECK(greater <= pos && pos < greater + equal);

    /* fused compress with the threshold left in the handle's slot */
    int bytes = 0;
    CHECK(cx_ip_compress(h, CX_F32, d_msg, cap, d_g, d_r, N, NULL, NULL, NULL, &bytes) == CX_OK);
    CHECK(bytes == 8 + 8 * greater);
    int bytes_read = 0;
    CHECK(cx_ip_decompress(h, CX_F32, d_dense, N, d_msg, &bytes_read) == CX_OK && bytes_read == bytes);
    CHECK(cx_copy(h, back, d_dense, N * sizeof(float)) == CX_OK);
    float* rest = malloc(N * sizeof(float));
    CHECK(cx_copy(h, rest, d_r, N * sizeof(float)) == CX_OK);
    CHECK(cx_synchronize(h) == CX_OK);
    for (int i = 0; i < N; ++i) {
        const float s = r[i] + g[i];
        const int sent = fabsf(s) > thr;
        if (back[i] != (sent ? s : 0.0f) || rest[i] != (sent ? 0.0f : s)) {
            ++errors;
            break;
        }
    }
    /* the same step as one call gives the same message */
    CHECK(cx_copy(h, d_r, r, N * sizeof(float)) == CX_OK);
    int bytes2 = 0;
    CHECK(cx_ip_compress_topk(h, CX_F32, d_msg, cap, d_g, d_r, N, topK, NULL, NULL, &bytes2) == CX_OK && bytes2 == bytes);
    /* add: dense += message */
    CHECK(cx_ip_add(h, CX_F32, d_dense, N, d_msg, 1) == CX_OK);
    CHECK(cx_copy(h, back, d_dense, N * sizeof(float)) == CX_OK);
    CHECK(cx_synchronize(h) == CX_OK);
    for (int i = 0; i < N; ++i) {
        const float s = r[i] + g[i];
        if (back[i] != (fabsf(s) > thr ? 2.0f * s : 0.0f)) {
            ++errors;
            break;
        }
    }
    /* run-length codec: |x| >= thr; decode gives the same dense vector once more */
    int rle_bytes = 0, n_msg = 0;
    CHECK(cx_rle_compress(h, CX_F32, d_rle, rle_cap, d_g, NULL, N, &thr, NULL, NULL, &rle_bytes) == CX_OK);
    CHECK(rle_bytes > 16 && rle_bytes <= rle_cap);
    CHECK(cx_rle_decompress(h, CX_F32, d_dense, N, d_rle, &n_msg) == CX_OK && n_msg == N);
    CHECK(cx_copy(h, back, d_dense, N * sizeof(float)) == CX_OK);
    CHECK(cx_synchronize(h) == CX_OK);
    for (int i = 0; i < N; ++i)
        if (back[i] != (fabsf(g[i]) >= thr ? g[i] : 0.0f)) {
            ++errors;
            break;
        }
    /* error paths: status codes instead of exceptions */
    CHECK(cx_topk_threshold(h, CX_F32, d_r, d_g, N, N - 1, topK, 1000, 10.0f, NULL, &thr) == CX_ERR_SIZE_MISMATCH);
    CHECK(cx_topk_threshold(h, CX_F32, d_r, NULL, N, 0, 1.5f, 1000, 10.0f, NULL, &thr) == CX_ERR_TOPK);
    CHECK(cx_ip_decompress(h, CX_F32, d_dense, N - 1, d_msg, &bytes_read) == CX_ERR_MSG_TOO_LARGE);
    const float zero = 0.0f;
    CHECK(cx_ip_compress(h, CX_F32, d_msg, 8 + 8 * 10, d_g, NULL, N, &zero, NULL, NULL, &bytes) == CX_ERR_CAPACITY);
    CHECK(strlen(cx_last_error()) > 0);
    CHECK(cx_set_option(h, "no_such_option", 1) == CX_ERR_INVALID);

    cx_device_free(d_g); cx_device_free(d_r); cx_device_free(d_msg); cx_device_free(d_dense); cx_device_free(d_rle);
    CHECK(cx_destroy(h) == CX_OK);
    free(g); free(r); free(back); free(rest);
    printf("kernel-level C ABI from plain C\n");
    if (errors == 0) printf("+++ PASSED +++\n");
    else printf("--- FAILED ---\nwith %d errors.\n", errors);
    return errors ? 1 : 0;
}
