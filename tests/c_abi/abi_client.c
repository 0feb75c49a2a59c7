/* A client of libneureka_hip.so written in plain C: what a JNI / Panama / cgo binding does, without any of
 * the Python mirror.  Exercises the lifecycle, memory and kernel entry points on tiny inputs and checks
 * every result on the host.  Built and run by tests/test_c_abi_client.py. */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "neureka_hip.h"

#define CHECK(call)                                                                      \
    do {                                                                                 \
        int status_ = (call);                                                            \
        if (status_ != 0) {                                                              \
            printf("FAIL %s -> %d: %s\n", #call, status_, nk_last_error());              \
            return 1;                                                                    \
        }                                                                                \
    } while (0)
#define EXPECT(cond)                                                                     \
    do {                                                                                 \
        if (!(cond)) { printf("FAIL line %d: %s\n", __LINE__, #cond); return 1; }        \
    } while (0)

/* dense row-major descriptor: shape | strides | indicesMap | offset | spread */
static void dense_cfg(int32_t* cfg, const int* shape, int rank) {
    int prod = 1;
    for (int k = rank - 1; k >= 0; k--) {
        cfg[0 * rank + k] = shape[k];
        cfg[1 * rank + k] = prod;
        cfg[2 * rank + k] = prod;
        cfg[3 * rank + k] = 0;
        cfg[4 * rank + k] = 1;
        prod *= shape[k];
    }
}

int main(void) {
    int count = 0;
    CHECK(nk_device_count(&count));
    EXPECT(count >= 1);
    nk_dev dev;
    CHECK(nk_device_open(0, &dev));
    char name[128];
    int cus = 0, wave = 0;
    CHECK(nk_device_props(dev, name, sizeof name, &cus, NULL, NULL, NULL, &wave));
    printf("device: %s, %d compute units, wavefront %d\n", name, cus, wave);
    EXPECT(wave == 64);

    /* broadcast add: [2,1,3] + [1,2,3] -> [2,2,3] */
    const int sa[3] = {2, 1, 3}, sb[3] = {1, 2, 3}, so[3] = {2, 2, 3};
    int32_t ca[15], cb[15], co[15];
    dense_cfg(ca, sa, 3); dense_cfg(cb, sb, 3); dense_cfg(co, so, 3);
    const float a[6] = {1, 2, 3, 4, 5, 6}, b[6] = {10, 20, 30, 40, 50, 60};
    float out[12];
    nk_buf da, db, dout;
    CHECK(nk_alloc(dev, sizeof a, &da)); CHECK(nk_alloc(dev, sizeof b, &db)); CHECK(nk_alloc(dev, sizeof out, &dout));
    CHECK(nk_h2d(dev, da, 0, a, sizeof a)); CHECK(nk_h2d(dev, db, 0, b, sizeof b));
    CHECK(nk_broadcast(dev, NK_OP_ADD, -1, NK_F32, 3, dout, co, da, ca, db, cb, 12));
    CHECK(nk_d2h(dev, out, dout, 0, sizeof out));
    for (int i = 0; i < 2; i++)
        for (int j = 0; j < 2; j++)
            for (int k = 0; k < 3; k++) EXPECT(out[(i * 2 + j) * 3 + k] == a[i * 3 + k] + b[j * 3 + k]);
    printf("broadcast add ok (%s)\n", nk_last_path());

    /* activation through a fill: tanh of a constant tensor */
    const float half = 0.5f;
    CHECK(nk_fill(dev, dout, 0, &half, 4, 12));
    CHECK(nk_activation(dev, NK_FUN_TANH, -1, NK_F32, 3, dout, co, dout, co, 12));
    CHECK(nk_d2h(dev, out, dout, 0, sizeof out));
    for (int i = 0; i < 12; i++) EXPECT(fabsf(out[i] - tanhf(0.5f)) <= 1e-5f * tanhf(0.5f));

    /* matmul: [2,3] @ [3,2], accumulated into a zeroed C */
    const float A[6] = {1, 2, 3, 4, 5, 6}, B[6] = {7, 8, 9, 10, 11, 12};
    float C[4] = {0, 0, 0, 0};
    nk_buf dA, dB, dC;
    CHECK(nk_alloc(dev, sizeof A, &dA)); CHECK(nk_alloc(dev, sizeof B, &dB)); CHECK(nk_alloc(dev, sizeof C, &dC));
    CHECK(nk_h2d(dev, dA, 0, A, sizeof A)); CHECK(nk_h2d(dev, dB, 0, B, sizeof B)); CHECK(nk_h2d(dev, dC, 0, C, sizeof C));
    CHECK(nk_matmul(dev, NK_F32, NK_LAYOUT_ROW_MAJOR, 2, 3, 2, dA, dB, dC));
    CHECK(nk_d2h(dev, C, dC, 0, sizeof C));
    EXPECT(C[0] == 58 && C[1] == 64 && C[2] == 139 && C[3] == 154);

    /* convolution [3,3] x [2,2] -> [2,2] (valid cross-correlation) */
    const int sx[2] = {3, 3}, sk[2] = {2, 2}, sy[2] = {2, 2};
    int32_t cx[10], ck[10], cy[10];
    dense_cfg(cx, sx, 2); dense_cfg(ck, sk, 2); dense_cfg(cy, sy, 2);
    const float x[9] = {1, 2, 3, 4, 5, 6, 7, 8, 9}, k[4] = {1, 0, 0, -1};
    float y[4];
    nk_buf dx, dk, dy;
    CHECK(nk_alloc(dev, sizeof x, &dx)); CHECK(nk_alloc(dev, sizeof k, &dk)); CHECK(nk_alloc(dev, sizeof y, &dy));
    CHECK(nk_h2d(dev, dx, 0, x, sizeof x)); CHECK(nk_h2d(dev, dk, 0, k, sizeof k));
    CHECK(nk_convolution(dev, -1, NK_F32, 2, dy, cy, dx, cx, dk, ck, 4));
    CHECK(nk_d2h(dev, y, dy, 0, sizeof y));
    EXPECT(y[0] == -4 && y[1] == -4 && y[2] == -4 && y[3] == -4);

    /* reductions */
    float total = 0;
    int32_t where = -1;
    nk_buf dsum, dwhere;
    CHECK(nk_alloc(dev, 4, &dsum)); CHECK(nk_alloc(dev, 4, &dwhere));
    CHECK(nk_sum(dev, NK_F32, dx, 9, dsum));
    CHECK(nk_d2h(dev, &total, dsum, 0, 4));
    EXPECT(total == 45);
    CHECK(nk_reduce_index(dev, NK_REDUCE_MAX, NK_F32, dx, 9, dwhere));
    CHECK(nk_d2h(dev, &where, dwhere, 0, 4));
    EXPECT(where == 8);

    /* integer scalarization: Java's int arithmetic (wrapping multiply, truncating division), / by zero is an error */
    const int32_t iv[5] = {2147483647, -7, 7, 0, -2147483647 - 1};
    int32_t ir[5];
    const int five[1] = {5};
    int32_t ci[5];
    dense_cfg(ci, five, 1);
    nk_buf di, dr;
    CHECK(nk_alloc(dev, sizeof iv, &di)); CHECK(nk_alloc(dev, sizeof ir, &dr));
    CHECK(nk_h2d(dev, di, 0, iv, sizeof iv));
    CHECK(nk_scalarization_int(dev, NK_OP_MUL, -1, NK_I32, 1, dr, ci, di, ci, 2, 5));
    CHECK(nk_d2h(dev, ir, dr, 0, sizeof ir));
    EXPECT(ir[0] == -2 && ir[1] == -14 && ir[2] == 14 && ir[3] == 0 && ir[4] == 0);
    CHECK(nk_scalarization_int(dev, NK_OP_DIV, -1, NK_I32, 1, dr, ci, di, ci, 2, 5));
    CHECK(nk_d2h(dev, ir, dr, 0, sizeof ir));
    EXPECT(ir[0] == 1073741823 && ir[1] == -3 && ir[2] == 3 && ir[3] == 0 && ir[4] == -1073741824);
    EXPECT(nk_scalarization_int(dev, NK_OP_DIV, -1, NK_I32, 1, dr, ci, di, ci, 0, 5) != 0);
    CHECK(nk_free(dev, di)); CHECK(nk_free(dev, dr));

    /* a descriptor that reaches outside its buffer is an error, not a launch */
    const int too_big[2] = {4, 4};
    int32_t cbad[10];
    dense_cfg(cbad, too_big, 2);
    EXPECT(nk_activation(dev, NK_FUN_RELU, -1, NK_F32, 2, dy, cbad, dy, cbad, 16) != 0);
    EXPECT(strlen(nk_last_error()) > 0);

    uint64_t live = 0, bytes = 0;
    CHECK(nk_device_stats(dev, &live, &bytes));
    EXPECT(live == 11);
    CHECK(nk_free(dev, da)); CHECK(nk_free(dev, db)); CHECK(nk_free(dev, dout));
    CHECK(nk_device_stats(dev, &live, &bytes));
    EXPECT(live == 8);
    CHECK(nk_device_close(dev));              /* releases what is still alive */
    printf("C ABI client: all checks passed\n");
    return 0;
}
