// nk_broadcast: forward broadcast (delegates to the elementwise engine) and the reducing backward.
//
// Backward (d >= 0), CPUBroadcast.java:207-259 (J/backend/main/implementations/broadcast/): the drain is
// the smaller tensor; per drain element the kernel sums g(src1, src2) over the axes on which the drain
// is smaller than src1, axis 0 fastest.  Every drain element is summed by one thread in the reference's
// order, so + and - results are bit-identical to the CPU device.
#include "nk_internal.h"
#include "nk_scalar.h"
#include <type_traits>

namespace nk {

int broadcast_forward(nk_dev dev, int op_id, int dtype, int rank, nk_buf drn, const int32_t* drn_cfg,
                      nk_buf a, const int32_t* a_cfg, nk_buf b, const int32_t* b_cfg, int64_t n);

// Physical offsets are linear in the nd-index (phys = sum (idx*spread + offset) * stride), so per launch the host
// reduces the three descriptors to: a base offset and one effective stride per axis for each operand as it
// follows the drain's index, plus the list of reduced axes (axis 0 first = fastest, the reference's order) with
// their extents and strides in src1 and src2.  A thread owns V drain elements that are neighbours along the
// last axis and walks the reduced axes with running offsets; the loads of UNROLL terms are requested together and
// then added in order, so the sum keeps the reference's order while the memory system sees deep queues.
struct BcastBwdArgs {
    int rank, op, d;
    unsigned n_threads;                  // drain elements / V
    int nred;
    Cfg c0;                              // the drain (flat index -> nd-index -> offset)
    int64_t base1, base2;
    int64_t keep1[NK_MAX_RANK], keep2[NK_MAX_RANK];       // stride of src1 / src2 along axis k as the drain's index moves (0: pinned)
    int red_extent[NK_MAX_RANK];
    int64_t red1[NK_MAX_RANK], red2[NK_MAX_RANK];
};

// The eight forms the backward term takes: CPUBroadcast<Op>.java _getDeriveAt0 / _getDeriveAt1 (these differ from
// the same-shape elementwise derivatives: the backward of + and - adds the operands because src1 is a zero tensor
// there).  The form is a template parameter, so the inner loop carries no operator dispatch, and an operand that
// is not part of the term is not read.
enum { G_SUM = 0, G_DIFF = 1, G_SECOND = 2, G_FIRST = 3, G_RCP = 4, G_DDIV = 5, G_DPOW_A = 6, G_DPOW_B = 7 };
static int derive_form(int op, int d) {
    switch (op) {
        case NK_OP_ADD: return G_SUM;
        case NK_OP_SUB: return d == 0 ? G_SUM : G_DIFF;
        case NK_OP_MUL: return d == 0 ? G_SECOND : G_FIRST;
        case NK_OP_DIV:
        case NK_OP_MOD: return d == 0 ? G_RCP : G_DDIV;
        default:        return d == 0 ? G_DPOW_A : G_DPOW_B;
    }
}
template <typename T, int G>
__device__ __forceinline__ T derive_term(T a, T b) {
    if constexpr (G == G_SUM) return a + b;
    if constexpr (G == G_DIFF) return a - b;
    if constexpr (G == G_SECOND) return b;
    if constexpr (G == G_FIRST) return a;
    if constexpr (G == G_RCP) return T(1) / b;
    if constexpr (G == G_DDIV) return ddiv_db_ref(a, b);
    if constexpr (G == G_DPOW_A) return bcast_dpow_da_ref(a, b);
    return dpow_db_ref(a, b);
}

template <typename T, int V, int G>
__global__ __launch_bounds__(256) void broadcast_bwd_kernel(BcastBwdArgs A, T* __restrict__ drn,
                                                            const T* __restrict__ s1, const T* __restrict__ s2) {
    constexpr int UNROLL = 8;
    typedef typename std::conditional<V == 1, T, T __attribute__((ext_vector_type(V == 1 ? 2 : V), aligned(sizeof(T))))>::type Vec;
    const unsigned t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= A.n_threads) return;
    int o[NK_MAX_RANK];
    nd_of_flat(A.c0, A.rank, (int)(t * V), o);
    int64_t o1 = A.base1, o2 = A.base2;
    for (int k = 0; k < A.rank; k++) { o1 += o[k] * A.keep1[k]; o2 += o[k] * A.keep2[k]; }
    T value[V];
#pragma unroll
    for (int v = 0; v < V; v++) value[v] = T(0);
    const int n0 = A.nred > 0 ? A.red_extent[0] : 1;
    const int64_t st1 = A.nred > 0 ? A.red1[0] : 0, st2 = A.nred > 0 ? A.red2[0] : 0;

    // PINNED: src1 does not move along the last axis (V > 1 only): one element serves the thread's V neighbours
    auto reduce = [&](auto pinned_tag) {
        constexpr bool PINNED = decltype(pinned_tag)::value;
        auto load1 = [&](int64_t at, T (&dst)[V]) {
            if constexpr (G == G_SECOND || G == G_RCP) { for (int v = 0; v < V; v++) dst[v] = T(0); }      // src1 is not part of the term
            else if constexpr (V == 1) dst[0] = s1[at];
            else if constexpr (PINNED) { const T x = s1[at]; for (int v = 0; v < V; v++) dst[v] = x; }
            else { const Vec x = *(const Vec*)(s1 + at); for (int v = 0; v < V; v++) dst[v] = ((const T*)&x)[v]; }
        };
        auto load2 = [&](int64_t at, T (&dst)[V]) {
            if constexpr (G == G_FIRST) { for (int v = 0; v < V; v++) dst[v] = T(0); }                     // src2 is not part of the term
            else if constexpr (V == 1) dst[0] = s2[at];
            else { const Vec x = __builtin_nontemporal_load((const Vec*)(s2 + at)); for (int v = 0; v < V; v++) dst[v] = ((const T*)&x)[v]; }
        };
        int r[NK_MAX_RANK];
        for (int k = 0; k < NK_MAX_RANK; k++) r[k] = 0;
        for (;;) {
            // the loads of the next UNROLL terms are issued before the current ones are added, so a wavefront
            // always has requests in flight; the order of the additions is the reference's
            int j = 0;
            const int batches = n0 / UNROLL;
            if (batches > 0) {
                T a[UNROLL][V], b[UNROLL][V], an[UNROLL][V], bn[UNROLL][V];
#pragma unroll
                for (int u = 0; u < UNROLL; u++) { load1(o1 + u * st1, a[u]); load2(o2 + u * st2, b[u]); }
                for (int bi = 0; bi < batches; bi++) {
                    if (bi + 1 < batches) {
                        const int64_t jn = (int64_t)(bi + 1) * UNROLL;
#pragma unroll
                        for (int u = 0; u < UNROLL; u++) { load1(o1 + (jn + u) * st1, an[u]); load2(o2 + (jn + u) * st2, bn[u]); }
                    }
#pragma unroll
                    for (int u = 0; u < UNROLL; u++)
#pragma unroll
                        for (int v = 0; v < V; v++) value[v] = value[v] + derive_term<T, G>(a[u][v], b[u][v]);
#pragma unroll
                    for (int u = 0; u < UNROLL; u++)
#pragma unroll
                        for (int v = 0; v < V; v++) { a[u][v] = an[u][v]; b[u][v] = bn[u][v]; }
                }
                j = batches * UNROLL;
            }
            for (; j < n0; j++) {
                T a[V], b[V];
                load1(o1 + j * st1, a); load2(o2 + j * st2, b);
#pragma unroll
                for (int v = 0; v < V; v++) value[v] = value[v] + derive_term<T, G>(a[v], b[v]);
            }
            // carry into the slower reduced axes
            int k = 1;
            for (; k < A.nred; k++) {
                r[k]++; o1 += A.red1[k]; o2 += A.red2[k];
                if (r[k] < A.red_extent[k]) break;
                o1 -= (int64_t)A.red_extent[k] * A.red1[k]; o2 -= (int64_t)A.red_extent[k] * A.red2[k];
                r[k] = 0;
            }
            if (k >= A.nred) break;
        }
    };
    if (V > 1 && A.keep1[A.rank - 1] == 0) reduce(std::true_type{});
    else reduce(std::false_type{});

    const int at = phys_of_nd(A.c0, A.rank, o);
    if (V == 1) drn[at] = value[0];
    else {
        Vec out;
        for (int v = 0; v < V; v++) ((T*)&out)[v] = value[v];
        *(Vec*)(drn + at) = out;
    }
}

}  // namespace nk

using namespace nk;

static bool env_vec_ok() {
    static const bool on = [] { const char* v = getenv("NK_BWD_VECTOR"); return !(v && v[0] == '0'); }();
    return on;
}

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
    A.rank = rank; A.op = op_id; A.d = d;
    Cfg c1, c2;
    load_cfg(A.c0, drn_cfg, rank); load_cfg(c1, a_cfg, rank); load_cfg(c2, b_cfg, rank);
    A.base1 = 0; A.base2 = 0; A.nred = 0;
    for (int k = 0; k < rank; k++) {
        const int e0 = A.c0.shape[k], e1 = c1.shape[k], e2 = c2.shape[k];
        const int64_t f1 = (int64_t)c1.spread[k] * c1.strides[k], f2 = (int64_t)c2.spread[k] * c2.strides[k];
        A.base1 += (int64_t)c1.offset[k] * c1.strides[k];
        A.base2 += (int64_t)c2.offset[k] * c2.strides[k];
        A.keep1[k] = 0; A.keep2[k] = 0;
        if (e0 == e1) { A.keep1[k] = f1; A.keep2[k] = e2 == 1 ? 0 : f2; }    // both follow the drain (src2 pinned if it has extent 1)
        else if (e0 > e1) { A.keep2[k] = f2; }                                // src1 pinned to 0
        else { A.red_extent[A.nred] = e1; A.red1[A.nred] = f1; A.red2[A.nred] = f2; A.nred++; }   // reduced: both walk 0 .. e1-1
    }
    // four (two) drain neighbours per thread when they are neighbours in memory for the drain and src2 and
    // neighbours or one value for src1, and the drain's flat index unravels row-major on the last axis
    constexpr int VB = 16;
    const int V = VB / eb, last = rank - 1;
    const bool vec = A.c0.shape[last] % V == 0 && A.c0.imap[last] == 1 && (int64_t)A.c0.spread[last] * A.c0.strides[last] == 1 &&
                     A.c0.shape[last] >= c1.shape[last] && A.keep2[last] == 1 && (A.keep1[last] == 1 || A.keep1[last] == 0) &&
                     env_vec_ok();
    A.n_threads = (unsigned)(vec ? n / V : n);
    const unsigned blocks = (A.n_threads + 255) / 256;
    set_path(vec ? "broadcast_backward_vec" : "broadcast_backward");
    auto go = [&](auto form) {
        constexpr int G = decltype(form)::value;
        if (dtype == NK_F32) {
            if (vec) hipLaunchKernelGGL((broadcast_bwd_kernel<float, 4, G>), dim3(blocks), dim3(256), 0, dev->stream, A, (float*)drn, (const float*)a, (const float*)b);
            else     hipLaunchKernelGGL((broadcast_bwd_kernel<float, 1, G>), dim3(blocks), dim3(256), 0, dev->stream, A, (float*)drn, (const float*)a, (const float*)b);
        } else {
            if (vec) hipLaunchKernelGGL((broadcast_bwd_kernel<double, 2, G>), dim3(blocks), dim3(256), 0, dev->stream, A, (double*)drn, (const double*)a, (const double*)b);
            else     hipLaunchKernelGGL((broadcast_bwd_kernel<double, 1, G>), dim3(blocks), dim3(256), 0, dev->stream, A, (double*)drn, (const double*)a, (const double*)b);
        }
    };
    switch (derive_form(op_id, d)) {
        case G_SUM: go(std::integral_constant<int, G_SUM>{}); break;
        case G_DIFF: go(std::integral_constant<int, G_DIFF>{}); break;
        case G_SECOND: go(std::integral_constant<int, G_SECOND>{}); break;
        case G_FIRST: go(std::integral_constant<int, G_FIRST>{}); break;
        case G_RCP: go(std::integral_constant<int, G_RCP>{}); break;
        case G_DDIV: go(std::integral_constant<int, G_DDIV>{}); break;
        case G_DPOW_A: go(std::integral_constant<int, G_DPOW_A>{}); break;
        default: go(std::integral_constant<int, G_DPOW_B>{}); break;
    }
    NK_HIP(hipGetLastError());
    return NK_OK;
}
