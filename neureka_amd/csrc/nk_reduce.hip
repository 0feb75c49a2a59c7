// nk_broadcast: forward broadcast (delegates to the elementwise engine) and the reducing backward.
//
// Backward (d >= 0), CPUBroadcast.java:207-259 (J/backend/main/implementations/broadcast/): the drain is
// the smaller tensor; per drain element the kernel sums g(src1, src2) over the axes on which the drain
// is smaller than src1, axis 0 fastest.  One thread per drain element with the sum in the reference's
// order, so + and - results are bit-identical to the CPU device.
#include "nk_internal.h"
#include "nk_scalar.h"

namespace nk {

int broadcast_forward(nk_dev dev, int op_id, int dtype, int rank, nk_buf drn, const int32_t* drn_cfg,
                      nk_buf a, const int32_t* a_cfg, nk_buf b, const int32_t* b_cfg, int64_t n);

// CPUBroadcast<Op>.java _getDeriveAt0 / _getDeriveAt1 (these differ from the same-shape elementwise
// derivatives: the backward of + and - adds the operands because src1 is a zero tensor there).
template <typename T>
__device__ __forceinline__ T bcast_derive(int op, int d, T a, T b) {
    using N = Num<T>;
    switch (op) {
        case NK_OP_ADD: return a + b;
        case NK_OP_SUB: return d == 0 ? a + b : a - b;
        case NK_OP_MUL: return d == 0 ? b : a;
        case NK_OP_DIV:
        case NK_OP_MOD: return d == 0 ? T(1) / b : -(a / (b * b));
        case NK_OP_POW: return d == 0 ? a * N::pow(a, b - T(1)) : N::pow(a, b) * N::log(a);
    }
    return T(NAN);
}

struct BcastBwdArgs {
    int rank, op, d;
    unsigned n;
    Cfg c0, c1, c2;
};

template <typename T>
__global__ __launch_bounds__(256) void broadcast_bwd_kernel(BcastBwdArgs A, T* __restrict__ drn,
                                                            const T* __restrict__ s1, const T* __restrict__ s2) {
    const unsigned step = gridDim.x * blockDim.x;
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < A.n; i += step) {
        int o[NK_MAX_RANK], i1[NK_MAX_RANK], i2[NK_MAX_RANK];
        nd_of_flat(A.c0, A.rank, (int)i, o);
        for (int k = 0; k < A.rank; k++) {
            const int e0 = A.c0.shape[k], e1 = A.c1.shape[k], e2 = A.c2.shape[k];
            if (e0 == e1) { i1[k] = o[k]; i2[k] = (e2 == 1) ? 0 : o[k]; }
            else if (e0 > e1) { i1[k] = 0; i2[k] = o[k]; }
            else { i1[k] = 0; i2[k] = 0; }     // reduced axis: walks 0 .. e1-1
        }
        T value = T(0);
        bool running = true;
        while (running) {
            value = value + bcast_derive<T>(A.op, A.d, s1[phys_of_nd(A.c1, A.rank, i1)], s2[phys_of_nd(A.c2, A.rank, i2)]);
            // odometer over the reduced axes, axis 0 fastest
            int k = 0;
            for (; k < A.rank; k++) {
                if (A.c0.shape[k] < A.c1.shape[k]) {
                    i1[k]++; i2[k]++;
                    if (i1[k] == A.c1.shape[k]) { i1[k] = 0; i2[k] = 0; }
                    else break;
                }
            }
            running = k < A.rank;
        }
        drn[phys_of_nd(A.c0, A.rank, o)] = value;
    }
}

}  // namespace nk

using namespace nk;

extern "C" int nk_broadcast(nk_dev h, int op_id, int d, int dtype, int rank, nk_buf drn, const int32_t* drn_cfg,
                            nk_buf a, const int32_t* a_cfg, nk_buf b, const int32_t* b_cfg, int64_t n) {
    NK_REQUIRE(op_id >= NK_OP_ADD && op_id <= NK_OP_POW, "nk_broadcast: unknown operator id %d", op_id);
    NK_REQUIRE(d >= -1 && d <= 1, "nk_broadcast: derivative index %d outside [-1, 1]", d);
    if (d < 0) return broadcast_forward(h, op_id, dtype, rank, drn, drn_cfg, a, a_cfg, b, b_cfg, n);

    NK_DEVICE(dev, h);
    NK_REQUIRE(dtype == NK_F32 || dtype == NK_F64, "nk_broadcast: unknown dtype %d", dtype);
    if (int e = check_cfg("nk_broadcast(drain)", drn_cfg, rank)) return e;
    if (int e = check_cfg("nk_broadcast(src1)", a_cfg, rank)) return e;
    if (int e = check_cfg("nk_broadcast(src2)", b_cfg, rank)) return e;
    int64_t size = 1;
    for (int k = 0; k < rank; k++) size *= drn_cfg[k];
    NK_REQUIRE(n == size && size < ((int64_t)1 << 31), "nk_broadcast: n = %lld but the drain holds %lld elements", (long long)n, (long long)size);
    for (int k = 0; k < rank; k++) {
        const int e0 = drn_cfg[k], e1 = a_cfg[k], e2 = b_cfg[k];
        // indices the kernel will form must stay inside src2: it walks 0..e1-1 on reduced axes and
        // follows the drain elsewhere
        if (e0 < e1) NK_REQUIRE(e2 >= e1, "nk_broadcast: axis %d is reduced over %d entries but src2 has only %d", k, e1, e2);
        else if (e0 == e1) NK_REQUIRE(e2 == 1 || e2 >= e0, "nk_broadcast: axis %d: src2 extent %d does not cover the drain's %d", k, e2, e0);
        else NK_REQUIRE(e2 >= e0, "nk_broadcast: axis %d: src2 extent %d does not cover the drain's %d", k, e2, e0);
    }
    const int eb = dtype_bytes(dtype);
    if (int e = check_extent(dev, "nk_broadcast(drain)", drn, drn_cfg, rank, eb)) return e;
    if (int e = check_extent(dev, "nk_broadcast(src1)", a, a_cfg, rank, eb)) return e;
    if (int e = check_extent(dev, "nk_broadcast(src2)", b, b_cfg, rank, eb)) return e;
    BcastBwdArgs A{};
    A.rank = rank; A.op = op_id; A.d = d; A.n = (unsigned)n;
    load_cfg(A.c0, drn_cfg, rank); load_cfg(A.c1, a_cfg, rank); load_cfg(A.c2, b_cfg, rank);
    unsigned blocks = (unsigned)((n + 255) / 256);
    if (blocks > 65536) blocks = 65536;
    set_path("broadcast_backward");
    if (dtype == NK_F32)
        hipLaunchKernelGGL(broadcast_bwd_kernel<float>, dim3(blocks), dim3(256), 0, dev->stream, A, (float*)drn, (const float*)a, (const float*)b);
    else
        hipLaunchKernelGGL(broadcast_bwd_kernel<double>, dim3(blocks), dim3(256), 0, dev->stream, A, (double*)drn, (const double*)a, (const double*)b);
    NK_HIP(hipGetLastError());
    return NK_OK;
}
