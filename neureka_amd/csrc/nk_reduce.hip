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
    // S = 2: a thread owns the drain elements at index i and i + extent / 2 of one kept axis along which src1 is
    // pinned, so every value of src1 it loads serves two sums; c0.imap then unravels the halved index space
    int64_t pair2, pair0;                // what the second element adds to the offset into src2 / into the drain
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

template <typename T, int V, int G, int S = 1>
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
    T value[S][V];
#pragma unroll
    for (int s = 0; s < S; s++)
#pragma unroll
        for (int v = 0; v < V; v++) value[s][v] = T(0);
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
            // the loads of the next UNROLL terms are requested before the current ones are added, so a wavefront
            // always has requests in flight; the order of the additions is the reference's.  Two sets of registers
            // take turns (no copies), and the offsets of the next term to request move by additions only.
            int64_t q1 = o1, q2 = o2;
            auto request = [&](T (&a)[UNROLL][V], T (&b)[S][UNROLL][V]) {
#pragma unroll
                for (int u = 0; u < UNROLL; u++) {
                    load1(q1, a[u]);
#pragma unroll
                    for (int s = 0; s < S; s++) load2(q2 + s * A.pair2, b[s][u]);
                    q1 += st1; q2 += st2;
                }
            };
            auto consume = [&](const T (&a)[UNROLL][V], const T (&b)[S][UNROLL][V]) {
#pragma unroll
                for (int u = 0; u < UNROLL; u++)
#pragma unroll
                    for (int s = 0; s < S; s++)
#pragma unroll
                        for (int v = 0; v < V; v++) value[s][v] = value[s][v] + derive_term<T, G>(a[u][v], b[s][u][v]);
            };
            const int batches = n0 / UNROLL;
            if (batches > 0) {
                T a0[UNROLL][V], b0[S][UNROLL][V], a1[UNROLL][V], b1[S][UNROLL][V];
                request(a0, b0);
                int bi = 0;
                for (; bi + 2 <= batches; bi += 2) {
                    request(a1, b1);
                    consume(a0, b0);
                    if (bi + 2 < batches) request(a0, b0);
                    consume(a1, b1);
                }
                if (bi < batches) consume(a0, b0);
            }
            for (int j = batches * UNROLL; j < n0; j++) {
                T a[V], b[S][V];
                load1(q1, a);
#pragma unroll
                for (int s = 0; s < S; s++) load2(q2 + s * A.pair2, b[s]);
                q1 += st1; q2 += st2;
#pragma unroll
                for (int s = 0; s < S; s++)
#pragma unroll
                    for (int v = 0; v < V; v++) value[s][v] = value[s][v] + derive_term<T, G>(a[v], b[s][v]);
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
#pragma unroll
    for (int s = 0; s < S; s++) {
        if (V == 1) drn[at + s * A.pair0] = value[s][0];
        else {
            Vec out;
            for (int v = 0; v < V; v++) ((T*)&out)[v] = value[s][v];
            *(Vec*)(drn + at + s * A.pair0) = out;
        }
    }
}

// ---- few outputs, long sums ---------------------------------------------------------------------------------
// One thread per drain element cannot feed the machine when a gradient has few elements (a bias: 512 sums of
// 131 072 terms) or when the reduced axis is the contiguous one (every thread would walk its own row).  Here a
// block owns OT neighbouring drain elements and one segment of their sums: its 256 threads are TL = 256 / OT lanes
// per element; lane l of segment s takes the terms s * TL + l, then every (segments * TL)-th -- terms enumerated
// with the last reduced axis fastest, the order memory runs in -- and the lanes meet in LDS.
//   ROWS = false (the drain keeps the innermost axis): OT = 64, neighbouring threads own neighbouring drain elements,
//                so a wavefront reads 64 neighbouring elements of the error per term;
//   ROWS = true  (the innermost axis is reduced): neighbouring threads own neighbouring terms, VT of them each
//                through one 16-byte load when the axis allows it; TL = 64 or 256 by the length of the sums.
// Several segments write partial sums that a second launch adds in segment order.  The terms are the
// reference's; their order is not: results agree norm-wise (1e-5 / 1e-12).
struct BwdSplitArgs {
    unsigned n_out, out_blocks;          // drain elements, blocks of OT of them
    unsigned terms, seg_terms;           // term units (VT terms each) per drain element and (host side) per segment
    int segments;
    int splat1;                          // VT > 1: src1 does not move along the innermost reduced axis
    int contiguous;                      // segment s owns the term units [s * seg_terms, (s + 1) * seg_terms) instead of every
                                         // segments-th group of TL: chosen when a block's step covers a contiguous piece of
                                         // memory, so that every block walks its own contiguous stretch front to back
};

template <typename T, int G, int OT, bool ROWS, int VW, bool SPLAT = false, bool FLAT = false, int PAIR = 1>
__global__ __launch_bounds__(256) void broadcast_bwd_split_kernel(BcastBwdArgs A, BwdSplitArgs S, T* __restrict__ drn, T* __restrict__ partial,
                                                                  const T* __restrict__ s1, const T* __restrict__ s2) {
    // VW: width of the 16-byte accesses -- ROWS: VW neighbouring terms of one drain element per load;
    // otherwise VW neighbouring drain elements per thread
    constexpr int TL = 256 / OT;                                 // term lanes per drain element (group)
    // FLAT: the reduced axes nest in both sources and were merged into one by the host, so a lane's offsets move by a
    // constant from term to term (no carries) -- the carry chain below costs about 40 vector instructions per load
    constexpr int U = FLAT ? 8 : 4;                              // loads in flight per lane
    constexpr int VA = SPLAT ? 1 : VW;                           // values kept per term of src1: one serves all VW when it
                                                                 // does not move along the vector (a template parameter: a
                                                                 // run-time test in the term loop costs a quarter of the rate)
    constexpr int NV = ROWS ? PAIR : VW;                         // running sums per thread
    // PAIR = 2 (ROWS only): the thread also owns the drain element that lies A.pair0 / A.pair2 further on along a kept
    // axis where src1 is pinned -- the same terms of src1 serve both sums (S.n_out counts the first elements only)
    static_assert(PAIR == 1 || (ROWS && OT == 1), "pairs of drain elements: one pair per block");
    typedef typename std::conditional<VW == 1, T, T __attribute__((ext_vector_type(VW == 1 ? 2 : VW), aligned(sizeof(T))))>::type Vec;
    __shared__ T part[NV][256];
    const int tid = threadIdx.x;
    const unsigned ob = blockIdx.x % S.out_blocks, seg = blockIdx.x / S.out_blocks;
    const unsigned oi = ROWS ? (unsigned)tid / TL : (unsigned)tid % OT;
    const unsigned tl = ROWS ? (unsigned)tid % TL : (unsigned)tid / OT;
    const unsigned out = ROWS ? ob * OT + oi : (ob * OT + oi) * NV;   // first (or only) drain element of the thread
    const bool live = out < S.n_out;
    int o[NK_MAX_RANK];
    nd_of_flat(A.c0, A.rank, (int)(live ? out : 0), o);
    int64_t o1 = A.base1, o2 = A.base2;
    for (int k = 0; k < A.rank; k++) { o1 += o[k] * A.keep1[k]; o2 += o[k] * A.keep2[k]; }
    // the segments interleave: segment s takes the term units s * TL + tl, then those segments * TL further on, so
    // that the blocks running at one time read one window of memory together -- or, `contiguous`, each its own stretch
    const unsigned first = S.contiguous ? seg * S.seg_terms : seg * TL;
    const unsigned stride = S.contiguous ? (unsigned)TL : (unsigned)S.segments * TL;
    const unsigned seg_end = first + S.seg_terms;
    const unsigned end = S.contiguous && seg_end < S.terms ? seg_end : S.terms;
    // mixed-radix position of the lane's first term unit and of its step, last reduced axis fastest; the two
    // offsets follow it by additions only: a step adds the offset of that many units, a carry out of axis k takes
    // the axis back to its start and moves axis k - 1 on by one (no multiplication in the term loop)
    int idx[NK_MAX_RANK], step[NK_MAX_RANK];
    int64_t fix1[NK_MAX_RANK], fix2[NK_MAX_RANK];
    int64_t a1 = o1, a2 = o2, delta1 = 0, delta2 = 0;
    {
        unsigned r = first + tl, q = stride;
        for (int k = A.nred - 1; k >= 0; k--) {
            const unsigned e = (unsigned)A.red_extent[k];
            idx[k] = (int)(r % e); r /= e;
            step[k] = (int)(q % e); q /= e;
            a1 += idx[k] * A.red1[k]; a2 += idx[k] * A.red2[k];
            delta1 += step[k] * A.red1[k]; delta2 += step[k] * A.red2[k];
            fix1[k] = (k > 0 ? A.red1[k - 1] : 0) - (int64_t)e * A.red1[k];
            fix2[k] = (k > 0 ? A.red2[k - 1] : 0) - (int64_t)e * A.red2[k];
        }
    }
    auto advance = [&]() {
        int carry = 0;
        a1 += delta1; a2 += delta2;
        if constexpr (FLAT) return;
        for (int k = A.nred - 1; k >= 0; k--) {
            idx[k] += step[k] + carry;
            carry = idx[k] >= A.red_extent[k];
            if (carry) { idx[k] -= A.red_extent[k]; a1 += fix1[k]; a2 += fix2[k]; }
        }
    };
    auto fetch = [&](T (&a)[VA], T (&b)[PAIR][VW]) {
#pragma unroll
        for (int v = 0; v < VA; v++) a[v] = T(0);
#pragma unroll
        for (int p = 0; p < PAIR; p++)
#pragma unroll
            for (int v = 0; v < VW; v++) b[p][v] = T(0);
        if constexpr (G != G_SECOND && G != G_RCP) {
            if constexpr (VA == 1) a[0] = s1[a1];
            else { const Vec x = *(const Vec*)(s1 + a1); for (int v = 0; v < VW; v++) a[v] = ((const T*)&x)[v]; }
        }
        if constexpr (G != G_FIRST) {
#pragma unroll
            for (int p = 0; p < PAIR; p++) {
                const int64_t at = a2 + p * A.pair2;
                if (VW == 1) b[p][0] = s2[at];
                else { const Vec x = __builtin_nontemporal_load((const Vec*)(s2 + at)); for (int v = 0; v < VW; v++) b[p][v] = ((const T*)&x)[v]; }
            }
        }
    };
    T value[NV];
#pragma unroll
    for (int v = 0; v < NV; v++) value[v] = T(0);
    auto add = [&](const T (&a)[VA], const T (&b)[PAIR][VW]) {
#pragma unroll
        for (int p = 0; p < PAIR; p++)
#pragma unroll
            for (int v = 0; v < VW; v++) {
                T& sum = value[ROWS ? p : v];
                sum = sum + derive_term<T, G>(a[VA == 1 ? 0 : v], b[p][v]);
            }
    };
    const unsigned t = first + tl;
    const unsigned mine = t < end ? (end - t + stride - 1) / stride : 0;   // term units of this lane
    unsigned i = 0;
    for (; i + U <= mine; i += U) {                                  // U loads requested together, added in that order
        T a[U][VA], b[U][PAIR][VW];
#pragma unroll
        for (int u = 0; u < U; u++) { fetch(a[u], b[u]); advance(); }
#pragma unroll
        for (int u = 0; u < U; u++) add(a[u], b[u]);
    }
    for (; i < mine; i++) {
        T a[VA], b[PAIR][VW];
        fetch(a, b); advance();
        add(a, b);
    }
#pragma unroll
    for (int v = 0; v < NV; v++) part[v][tid] = live ? value[v] : T(0);
    __syncthreads();
    if (ROWS) {
        for (int w = TL / 2; w >= 1; w >>= 1) {
            if ((int)tl < w)
#pragma unroll
                for (int v = 0; v < NV; v++) part[v][tid] = part[v][tid] + part[v][tid + w];
            __syncthreads();
        }
    } else {
        for (int w = 128; w >= OT; w >>= 1) {
            if (tid < w)
#pragma unroll
                for (int v = 0; v < NV; v++) part[v][tid] = part[v][tid] + part[v][tid + w];
            __syncthreads();
        }
    }
    if (tl == 0 && live) {
        if (ROWS) {
#pragma unroll
            for (int p = 0; p < PAIR; p++) {     // partial sums: all first elements of a segment, then all second ones
                if (S.segments == 1) drn[phys_of_nd(A.c0, A.rank, o) + p * A.pair0] = part[p][tid];
                else partial[((int64_t)seg * PAIR + p) * S.n_out + out] = part[p][tid];
            }
        } else {
            T* dst = S.segments == 1 ? drn + phys_of_nd(A.c0, A.rank, o) : partial + (int64_t)seg * S.n_out + out;
#pragma unroll
            for (int v = 0; v < NV; v++) dst[v] = part[v][tid];      // NV > 1: the drain is contiguous along these elements
        }
    }
}

// partial[segment][element] -> drain: sixteen lanes per element take every sixteenth segment and meet in LDS
template <typename T>
__global__ __launch_bounds__(256) void broadcast_bwd_segments_kernel(Cfg c0, int rank, unsigned n_out, int segments, const T* __restrict__ partial,
                                                                     T* __restrict__ drn, unsigned firsts, int64_t pair0) {
    // n_out = firsts, or 2 * firsts when the blocks summed pairs of drain elements: element e >= firsts is the partner of
    // e - firsts, pair0 further on in the drain
    __shared__ T part[256];
    const int tid = threadIdx.x;
    const unsigned lane = (unsigned)tid & 15u, out = blockIdx.x * 16u + ((unsigned)tid >> 4);
    T s = T(0);
    if (out < n_out) {
        // eight loads requested together: with one at a time 2048 segments cost 128 memory latencies (44 us)
        int k = (int)lane;
        for (; k + 7 * 16 < segments; k += 8 * 16) {
            T v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = partial[(int64_t)(k + 16 * u) * n_out + out];
#pragma unroll
            for (int u = 0; u < 8; u++) s = s + v[u];
        }
        for (; k < segments; k += 16) s = s + partial[(int64_t)k * n_out + out];
    }
    part[tid] = s;
    __syncthreads();
    for (int w = 8; w >= 1; w >>= 1) {
        if ((int)lane < w) part[tid] = part[tid] + part[tid + w];
        __syncthreads();
    }
    if (lane == 0 && out < n_out) drn[out < firsts ? phys_of_flat(c0, rank, (int)out) : phys_of_flat(c0, rank, (int)(out - firsts)) + pair0] = part[tid];
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
    A.rank = rank; A.op = op_id; A.d = d;
    Cfg c1, c2;
    load_cfg(A.c0, drn_cfg, rank); load_cfg(c1, a_cfg, rank); load_cfg(c2, b_cfg, rank);
    tame_unravel(A.c0, rank, n);            // (the sources follow the drain's nd-index: their tables play no role)
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
                     A.c0.shape[last] >= c1.shape[last] && A.keep2[last] == 1 && (A.keep1[last] == 1 || A.keep1[last] == 0);
    A.n_threads = (unsigned)(vec ? n / V : n);
    // few outputs with long sums, or the innermost axis reduced: the kernel that splits the sums (another order of
    // the same terms, see above); everything else keeps the reference's order bit for bit
    int64_t terms = 1;
    for (int k = 0; k < A.nred; k++) terms *= A.red_extent[k];
    const bool last_reduced = A.c0.shape[last] < c1.shape[last];
    if (terms < ((int64_t)1 << 31) && ((last_reduced && terms >= 512) || (terms >= 1024 && A.n_threads < 16384))) {
        // innermost reduced axis in 16-byte pieces when it is contiguous in the error and contiguous or constant in src1
        int VT = 1;
        if (last_reduced) {
            const int lr = A.nred - 1;
            if (A.red_extent[lr] % V == 0 && A.red2[lr] == 1 && (A.red1[lr] == 1 || A.red1[lr] == 0)) VT = V;
        }
        const int64_t units = terms / VT;
        const int VO = !last_reduced && vec ? V : 1;                               // neighbouring drain elements per thread
        // lanes per drain element: by the length of the sums when the innermost axis is reduced; otherwise more lanes
        // the fewer drain elements there are, so that the blocks of at most 256 segments still fill the machine
        const int64_t out_threads = n / VO;
        // (a drain that is one row of 128 threads gets two rows per block: the block then reads whole rows)
        const int TL = last_reduced ? (units >= 2048 ? 256 : (units >= 512 ? 64 : 16)) : (out_threads >= 1024 ? 4 : (out_threads == 128 ? 2 : 16));
        const int OT = 256 / TL;
        BwdSplitArgs S{};
        S.n_out = (unsigned)n; S.terms = (unsigned)units;
        S.splat1 = last_reduced ? (VT > 1 && A.red1[A.nred - 1] == 0) : (A.keep1[last] == 0);
        if (VT > 1) { A.red_extent[A.nred - 1] /= VT; A.red1[A.nred - 1] *= VT; A.red2[A.nred - 1] *= VT; }
        // neighbouring reduced axes that nest in both sources (the slower one's stride is the faster one's whole
        // length) are one axis to the term enumeration, which runs last axis fastest
        for (int k = A.nred - 1; k > 0; k--) {
            if (A.red1[k - 1] == (int64_t)A.red_extent[k] * A.red1[k] && A.red2[k - 1] == (int64_t)A.red_extent[k] * A.red2[k] &&
                (int64_t)A.red_extent[k - 1] * A.red_extent[k] < ((int64_t)1 << 31)) {
                A.red_extent[k - 1] *= A.red_extent[k]; A.red1[k - 1] = A.red1[k]; A.red2[k - 1] = A.red2[k];
                for (int m = k; m + 1 < A.nred; m++) { A.red_extent[m] = A.red_extent[m + 1]; A.red1[m] = A.red1[m + 1]; A.red2[m] = A.red2[m + 1]; }
                A.nred--;
            }
        }
        const bool flat = A.nred == 1;
        // a step of the block is one contiguous piece of the error when its lanes take neighbouring 16-byte units of a
        // contiguous reduced axis (256 of them: 4 KiB), or when the block covers whole rows that follow each other
        // long sums over a contiguous innermost axis with src1 pinned along a kept axis (per-slab sums of a broadcast
        // operand): a block owns the two drain elements that lie half that axis apart and reads src1 once for both
        A.pair2 = 0; A.pair0 = 0;
        int pairs = 1;
        const int form_of_term = derive_form(op_id, d);
        if (flat && last_reduced && TL == 256 && VT > 1 && !S.splat1 && form_of_term != G_SECOND && form_of_term != G_RCP && n >= 512) {
            bool row_major = true;
            int64_t run = 1;
            for (int k = rank - 1; k >= 0; k--) { if (A.c0.shape[k] > 1 && A.c0.imap[k] != run) row_major = false; run *= A.c0.shape[k]; }
            for (int k = 0; row_major && pairs == 1 && k < rank; k++) {
                const int e = A.c0.shape[k];
                if (e >= 2 && e % 2 == 0 && A.keep1[k] == 0 && A.keep2[k] != 0) {
                    A.pair2 = (int64_t)(e / 2) * A.keep2[k];
                    A.pair0 = (int64_t)(e / 2) * A.c0.spread[k] * A.c0.strides[k];
                    A.c0.shape[k] = e / 2;
                    int64_t m = 1;
                    for (int j = rank - 1; j >= 0; j--) { A.c0.imap[j] = (int)m; m *= A.c0.shape[j]; }
                    pairs = 2;
                }
            }
        }
        const int64_t firsts = n / pairs;                                             // drain elements the blocks enumerate
        S.n_out = (unsigned)firsts;
        S.out_blocks = (unsigned)((firsts / VO + OT - 1) / OT);
        S.contiguous = flat && (last_reduced ? (TL == 256 && VT > 1) : (S.out_blocks == 1 && VO > 1 && A.red2[0] == n));
        // enough blocks to fill the machine: eight per compute unit where the segments interleave; where every block
        // walks its own contiguous stretch, few long-running blocks read fastest (bias gradient of 4 GiB: 2048 blocks
        // 6.7, 1024 6.9, 512 7.1, 256 7.2 TB/s) ...
        const int64_t want_blocks = S.contiguous ? 2 * dev->props.multiProcessorCount : 2048;
        int64_t segs = (want_blocks + S.out_blocks - 1) / S.out_blocks;
        const int64_t most = units / (TL * 8) > 0 ? units / (TL * 8) : 1;         // ... with at least 8 term units per lane
        if (segs > most) segs = most;
        if (segs > 256) segs = 256;
        if (segs < 1) segs = 1;
        S.seg_terms = (unsigned)((units + segs - 1) / segs);
        S.segments = (int)((units + S.seg_terms - 1) / S.seg_terms);
        void* ws = nullptr;
        if (S.segments > 1)
            if (int e = workspace(dev, (uint64_t)S.segments * n * eb, &ws)) return e;
        const unsigned grid = S.out_blocks * (unsigned)S.segments;
        set_path(last_reduced ? (pairs == 2 ? "broadcast_backward_split_rows_vec_pairs" : VT > 1 ? "broadcast_backward_split_rows_vec" : "broadcast_backward_split_rows")
                              : (VO > 1 ? "broadcast_backward_split_vec" : "broadcast_backward_split"));
        auto split = [&](auto form) {
            constexpr int G = decltype(form)::value;
            auto typed = [&](auto zero) {
                using T = decltype(zero);
                constexpr int VM = 16 / sizeof(T);
                T* d_ = (T*)drn; T* w_ = (T*)ws; const T* a_ = (const T*)a; const T* b_ = (const T*)b;
                if (!last_reduced) {
                    auto keep = [&](auto ot, auto vw) {
                        constexpr int O = decltype(ot)::value, W = decltype(vw)::value;
                        auto run = [&](auto splat, auto flat_tag) {
                            hipLaunchKernelGGL((broadcast_bwd_split_kernel<T, G, O, false, W, decltype(splat)::value, decltype(flat_tag)::value>), dim3(grid), dim3(256), 0, dev->stream, A, S, d_, w_, a_, b_);
                        };
                        if (W > 1 && S.splat1) { if (flat) run(std::true_type{}, std::true_type{}); else run(std::true_type{}, std::false_type{}); }
                        else { if (flat) run(std::false_type{}, std::true_type{}); else run(std::false_type{}, std::false_type{}); }
                    };
                    using one = std::integral_constant<int, 1>; using wide = std::integral_constant<int, VM>;
                    if (OT == 128) { if (VO > 1) keep(std::integral_constant<int, 128>{}, wide{}); else keep(std::integral_constant<int, 128>{}, one{}); }
                    else if (OT == 64) { if (VO > 1) keep(std::integral_constant<int, 64>{}, wide{}); else keep(std::integral_constant<int, 64>{}, one{}); }
                    else { if (VO > 1) keep(std::integral_constant<int, 16>{}, wide{}); else keep(std::integral_constant<int, 16>{}, one{}); }
                }
                else {
                    auto rows = [&](auto ot, auto vw, auto splat) {
                        if (pairs == 2) {
                            if constexpr (decltype(ot)::value == 1 && decltype(vw)::value == VM && !decltype(splat)::value)
                                hipLaunchKernelGGL((broadcast_bwd_split_kernel<T, G, 1, true, VM, false, true, 2>), dim3(grid), dim3(256), 0, dev->stream, A, S, d_, w_, a_, b_);
                        }
                        else if (flat) hipLaunchKernelGGL((broadcast_bwd_split_kernel<T, G, decltype(ot)::value, true, decltype(vw)::value, decltype(splat)::value, true>), dim3(grid), dim3(256), 0, dev->stream, A, S, d_, w_, a_, b_);
                        else      hipLaunchKernelGGL((broadcast_bwd_split_kernel<T, G, decltype(ot)::value, true, decltype(vw)::value, decltype(splat)::value, false>), dim3(grid), dim3(256), 0, dev->stream, A, S, d_, w_, a_, b_);
                    };
                    auto lanes = [&](auto ot) {
                        if (VT > 1 && S.splat1) rows(ot, std::integral_constant<int, VM>{}, std::true_type{});
                        else if (VT > 1) rows(ot, std::integral_constant<int, VM>{}, std::false_type{});
                        else rows(ot, std::integral_constant<int, 1>{}, std::false_type{});
                    };
                    if (TL == 256) lanes(std::integral_constant<int, 1>{});
                    else if (TL == 64) lanes(std::integral_constant<int, 4>{});
                    else lanes(std::integral_constant<int, 16>{});
                }
                if (S.segments > 1)
                    hipLaunchKernelGGL(broadcast_bwd_segments_kernel<T>, dim3((unsigned)((n + 15) / 16)), dim3(256), 0, dev->stream, A.c0, rank, (unsigned)n, S.segments, (const T*)ws, d_,
                                       S.n_out, A.pair0);
            };
            if (dtype == NK_F32) typed(0.0f); else typed(0.0);
        };
        switch (derive_form(op_id, d)) {
            case G_SUM: split(std::integral_constant<int, G_SUM>{}); break;
            case G_DIFF: split(std::integral_constant<int, G_DIFF>{}); break;
            case G_SECOND: split(std::integral_constant<int, G_SECOND>{}); break;
            case G_FIRST: split(std::integral_constant<int, G_FIRST>{}); break;
            case G_RCP: split(std::integral_constant<int, G_RCP>{}); break;
            case G_DDIV: split(std::integral_constant<int, G_DDIV>{}); break;
            case G_DPOW_A: split(std::integral_constant<int, G_DPOW_A>{}); break;
            default: split(std::integral_constant<int, G_DPOW_B>{}); break;
        }
        NK_HIP(hipGetLastError());
        return NK_OK;
    }
    // Two drain elements per thread where src1 is pinned along a kept axis (the forward broadcast repeated it there):
    // each value of src1 is then loaded once for two sums, which takes a quarter off the requests the vector memory
    // unit has to serve.  Needs the row-major unravelling of the drain's flat index and enough threads left.
    A.pair2 = 0; A.pair0 = 0;
    bool paired = false;
    if (vec && A.n_threads / 2 >= 256u * (unsigned)dev->props.multiProcessorCount) {
        bool row_major = true;
        int64_t run = 1;
        for (int k = rank - 1; k >= 0; k--) { if (A.c0.shape[k] > 1 && A.c0.imap[k] != run) row_major = false; run *= A.c0.shape[k]; }
        for (int k = 0; row_major && !paired && k < rank - 1; k++) {
            const int e = A.c0.shape[k];
            if (e >= 2 && e % 2 == 0 && A.keep1[k] == 0 && A.keep2[k] != 0) {
                A.pair2 = (int64_t)(e / 2) * A.keep2[k];
                A.pair0 = (int64_t)(e / 2) * A.c0.spread[k] * A.c0.strides[k];
                A.c0.shape[k] = e / 2;
                int64_t m = 1;
                for (int j = rank - 1; j >= 0; j--) { A.c0.imap[j] = (int)m; m *= A.c0.shape[j]; }
                A.n_threads /= 2;
                paired = true;
            }
        }
    }
    const unsigned blocks = (A.n_threads + 255) / 256;
    set_path(vec ? (paired ? "broadcast_backward_vec_pairs" : "broadcast_backward_vec") : "broadcast_backward");
    auto go = [&](auto form) {
        constexpr int G = decltype(form)::value;
        if (paired) {
            if (dtype == NK_F32) hipLaunchKernelGGL((broadcast_bwd_kernel<float, 4, G, 2>), dim3(blocks), dim3(256), 0, dev->stream, A, (float*)drn, (const float*)a, (const float*)b);
            else                 hipLaunchKernelGGL((broadcast_bwd_kernel<double, 2, G, 2>), dim3(blocks), dim3(256), 0, dev->stream, A, (double*)drn, (const double*)a, (const double*)b);
            return;
        }
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
