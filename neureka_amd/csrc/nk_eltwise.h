// Device side of the elementwise kernel family (activation, binary elementwise, scalarization, fill,
// forward broadcast, fused expressions): "drain[i] = program(sources at i)".
//
// The host (nk_eltwise.hip) compiles each operation to a small accumulator program and reduces the view
// descriptors to one of four access patterns; the kernels here are instantiated per
//   T        float | double
//   FUNSET   0: + - * / and copies only   1: + the cheap forward activations   2: the full table
//   NSRC     number of source registers the instantiation carries (1, 2, 3 or 6)
// so that the bandwidth-critical cases (add/mul, broadcast, the sig/tanh chain) run in kernels with a
// small register footprint, while rarely used functions live in their own, heavier instantiations.
#pragma once
#include "nk_internal.h"
#include "nk_scalar.h"

namespace nk {

// ---- accumulator programs ------------------------------------------------------------------------
enum : int { I_SET = 0, I_FUN, I_DFUN, I_BIN, I_RBIN, I_DBIN, I_RDBIN, I_PUSH };
constexpr int SRC_CONST0 = 16, SRC_POP = 32;
constexpr int MAX_INSTR = 48;
constexpr int HW_STACK = 4;

struct Prog {
    int n;
    unsigned char op[MAX_INSTR];   // I_*
    unsigned char arg[MAX_INSTR];  // fun id | binary op | (binary op)*2 + d
    unsigned char src[MAX_INSTR];  // k | SRC_CONST0 + k | SRC_POP
    double consts[NK_FUSE_MAX_CONST];
};

// interpreter: V elements per thread; all control flow is uniform over the grid (it only depends on
// kernel arguments), so it costs scalar branches, not divergence.
// Only the full function set (FUNSET 2) carries the four-deep stack of saved intermediates; programs
// that need it are routed there by the host.
template <typename T, int V, int NSRC, int FUNSET>
__device__ __forceinline__ void run_prog(const Prog& P, const T (&src)[NSRC][V], T (&acc)[V]) {
    constexpr bool STACK = FUNSET >= 2;
    constexpr int SV = STACK ? V : 1;
    T s0[SV], s1[SV], s2[SV], s3[SV];
#pragma unroll
    for (int v = 0; v < V; v++) acc[v] = T(0);
#pragma unroll
    for (int v = 0; v < SV; v++) s0[v] = s1[v] = s2[v] = s3[v] = T(0);
    for (int pc = 0; pc < P.n; pc++) {
        const int op = P.op[pc], arg = P.arg[pc], s = P.src[pc];
        T x[V];
        if (op == I_PUSH) {
            if constexpr (STACK) {
#pragma unroll
                for (int v = 0; v < V; v++) { s3[v] = s2[v]; s2[v] = s1[v]; s1[v] = s0[v]; s0[v] = acc[v]; }
            }
            continue;
        }
        if (op != I_FUN && op != I_DFUN) {
            if (STACK && s == SRC_POP) {
                if constexpr (STACK) {
#pragma unroll
                    for (int v = 0; v < V; v++) { x[v] = s0[v]; s0[v] = s1[v]; s1[v] = s2[v]; s2[v] = s3[v]; }
                }
            } else if (s >= SRC_CONST0) {
                T c = (T)P.consts[s - SRC_CONST0];
#pragma unroll
                for (int v = 0; v < V; v++) x[v] = c;
            } else {
#pragma unroll
                for (int v = 0; v < V; v++) x[v] = src[0][v];
#pragma unroll
                for (int j = 1; j < NSRC; j++)
                    if (s == j) {
#pragma unroll
                        for (int v = 0; v < V; v++) x[v] = src[j][v];
                    }
            }
        }
        switch (op) {
            case I_SET:
#pragma unroll
                for (int v = 0; v < V; v++) acc[v] = x[v];
                break;
            case I_FUN:
                if constexpr (FUNSET >= 1) apply_fun<T, V, FUNSET>(arg, acc);
                break;
            case I_DFUN:
                if constexpr (FUNSET >= 2) apply_dfun<T, V>(arg, acc);
                break;
            case I_BIN: apply_bin<T, V, FUNSET>(arg, acc, x); break;
            case I_RBIN:
                apply_bin<T, V, FUNSET>(arg, x, acc);
#pragma unroll
                for (int v = 0; v < V; v++) acc[v] = x[v];
                break;
            case I_DBIN: apply_dbin<T, V, FUNSET>(arg >> 1, arg & 1, acc, x); break;
            case I_RDBIN:
                apply_dbin<T, V, FUNSET>(arg >> 1, arg & 1, x, acc);
#pragma unroll
                for (int v = 0; v < V; v++) acc[v] = x[v];
                break;
        }
    }
}

// ---- helpers ---------------------------------------------------------------------------------------
// unsigned division by an invariant divisor, valid for numerators below 2^31
struct FastDiv {
    unsigned d = 1, mul = 0, shift = 0;
    FastDiv() = default;
    explicit FastDiv(unsigned div) : d(div) {
        if (div <= 1) { mul = 0; shift = 0; return; }
        unsigned l = 0;
        while ((1u << l) < div) l++;                 // ceil(log2(div))
        uint64_t p = 31 + l;
        mul = (unsigned)((((uint64_t)1 << p) + div - 1) / div);
        shift = (unsigned)(p - 32);
    }
    __host__ __device__ __forceinline__ unsigned div(unsigned n) const {
#if defined(__HIP_DEVICE_COMPILE__)
        return d == 1 ? n : (__umulhi(n, mul) >> shift);
#else
        return d == 1 ? n : (unsigned)(((uint64_t)n * mul) >> 32) >> shift;
#endif
    }
};

struct Ptrs { const void* p[NK_FUSE_MAX_SRC]; };

template <typename T, int V> struct VecOf { typedef T type __attribute__((ext_vector_type(V))); };
template <typename T> struct VecOf<T, 1> { typedef T type; };

template <typename T, int V>
__device__ __forceinline__ void load_vec(T (&dst)[V], const T* p) {
    if constexpr (V == 1) dst[0] = *p;
    else {
        typename VecOf<T, V>::type v = *(const typename VecOf<T, V>::type*)p;
#pragma unroll
        for (int i = 0; i < V; i++) dst[i] = v[i];
    }
}
template <typename T, int V>
__device__ __forceinline__ void store_vec(T* p, const T (&src)[V], bool streaming) {
    if constexpr (V == 1) {
        if (streaming) __builtin_nontemporal_store(src[0], p); else *p = src[0];
    } else {
        typename VecOf<T, V>::type v;
#pragma unroll
        for (int i = 0; i < V; i++) v[i] = src[i];
        if (streaming) __builtin_nontemporal_store(v, (typename VecOf<T, V>::type*)p);
        else *(typename VecOf<T, V>::type*)p = v;
    }
}

// ---- rows kernel -----------------------------------------------------------------------------------
// Every operand is contiguous (stride 1) or constant (stride 0) along the innermost collapsed axis.
// A block of 256 threads covers `256 >> tpr_log2` rows per pass and PASSES passes per tile; a thread
// issues the loads of all its passes before it computes and stores, so that several 16-byte requests
// per source are in flight per lane.
struct RowsArgs {
    int rank;                  // collapsed rank >= 1
    int nsrc;
    unsigned L;                // innermost extent
    unsigned n_rows;           // product of the outer extents
    int tpr_log2;              // threads per row, log2
    unsigned chunks;           // column chunks per row
    unsigned n_tiles;
    unsigned scalar_load;      // bit j: source j is not 16-byte aligned: element-wise loads
    int streaming;             // non-temporal stores for the drain
    FastDiv chunk_div;
    FastDiv outer[NK_MAX_RANK];             // outer[k] divides by shape[k], k < rank-1
    int64_t base[MAX_OPERANDS];
    int64_t stride[MAX_OPERANDS][NK_MAX_RANK];
};

template <typename T, int V, int NSRC, int FUNSET, int PASSES>
__global__ __launch_bounds__(256) void rows_kernel(RowsArgs A, Prog P, T* __restrict__ drn, Ptrs srcs) {
    const unsigned tpr = 1u << A.tpr_log2;
    const unsigned rows_per_pass = 256u >> A.tpr_log2;
    const unsigned sub = threadIdx.x >> A.tpr_log2, lane = threadIdx.x & (tpr - 1);
    const int last = A.rank - 1;
    for (unsigned tile = blockIdx.x; tile < A.n_tiles; tile += gridDim.x) {
        const unsigned row_tile = A.chunk_div.div(tile);
        const unsigned chunk = tile - row_tile * A.chunks;
        const unsigned col = (chunk * tpr + lane) * V;
        if (col >= A.L) continue;
        T x[PASSES][NSRC][V];
        int64_t doff[PASSES];
        bool live[PASSES];
#pragma unroll
        for (int p = 0; p < PASSES; p++) {
            const unsigned row = (row_tile * PASSES + p) * rows_per_pass + sub;
            live[p] = row < A.n_rows;
            int64_t off[NSRC + 1];
#pragma unroll
            for (int o = 0; o <= NSRC; o++) off[o] = A.base[o];
            unsigned r = live[p] ? row : 0;
            for (int k = last - 1; k >= 0; k--) {
                const unsigned q = A.outer[k].div(r);
                const unsigned idx = r - q * A.outer[k].d;
                r = q;
#pragma unroll
                for (int o = 0; o <= NSRC; o++) off[o] += (int64_t)idx * A.stride[o][k];
            }
            doff[p] = off[0] + col;
#pragma unroll
            for (int j = 0; j < NSRC; j++) {
                if (j < A.nsrc && live[p]) {
                    const T* sp = (const T*)srcs.p[j] + off[j + 1];
                    if (A.stride[j + 1][last] == 0) {
                        const T c = *sp;
#pragma unroll
                        for (int v = 0; v < V; v++) x[p][j][v] = c;
                    } else if ((A.scalar_load >> j) & 1u) {
#pragma unroll
                        for (int v = 0; v < V; v++) x[p][j][v] = sp[col + v];
                    } else {
                        load_vec<T, V>(x[p][j], sp + col);
                    }
                } else {
#pragma unroll
                    for (int v = 0; v < V; v++) x[p][j][v] = T(0);
                }
            }
        }
#pragma unroll
        for (int p = 0; p < PASSES; p++) {
            if (live[p]) {
                T out[V];
                run_prog<T, V, NSRC, FUNSET>(P, x[p], out);
                store_vec<T, V>(drn + doff[p], out, A.streaming != 0);
            }
        }
    }
}

// ---- canon kernel: arbitrary strides, one element per thread -------------------------------------------
struct CanonArgs {
    int rank;
    int nsrc;
    unsigned n;
    FastDiv dims[NK_MAX_RANK];
    int64_t base[MAX_OPERANDS];
    int64_t stride[MAX_OPERANDS][NK_MAX_RANK];
};

template <typename T, int NSRC, int FUNSET>
__global__ __launch_bounds__(256) void canon_kernel(CanonArgs A, Prog P, T* __restrict__ drn, Ptrs srcs) {
    const unsigned step = gridDim.x * blockDim.x;
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < A.n; i += step) {
        int64_t off[NSRC + 1];
#pragma unroll
        for (int o = 0; o <= NSRC; o++) off[o] = A.base[o];
        unsigned r = i;
        for (int k = A.rank - 1; k >= 0; k--) {
            const unsigned q = A.dims[k].div(r);
            const unsigned idx = r - q * A.dims[k].d;
            r = q;
#pragma unroll
            for (int o = 0; o <= NSRC; o++) off[o] += (int64_t)idx * A.stride[o][k];
        }
        T x[NSRC][1];
#pragma unroll
        for (int j = 0; j < NSRC; j++) x[j][0] = j < A.nsrc ? ((const T*)srcs.p[j])[off[j + 1]] : T(0);
        T out[1];
        run_prog<T, 1, NSRC, FUNSET>(P, x, out);
        drn[off[0]] = out[0];
    }
}

// ---- tile_transpose kernel ----------------------------------------------------------------------------
// Collapsed axis `pax` (not the innermost) is the contiguous one of the sources flagged in `turned`; all
// other operands are contiguous or constant along the innermost axis.  A block owns a 64 (pax) x 64
// (innermost) tile for one combination of the remaining axes; turned sources are read with lanes along
// pax and handed to the lanes along the innermost axis through a padded LDS tile.
struct TileArgs {
    int rank;
    int nsrc;
    int pax;
    unsigned turned;                        // bit j: source j is read along pax
    unsigned P, L;                          // extents of pax and of the innermost axis
    unsigned tiles_p, tiles_l;
    unsigned n_blocks;
    int streaming;
    FastDiv div_tiles_l, div_tiles_p;
    FastDiv outer[NK_MAX_RANK];             // extents of the remaining axes
    int64_t base[MAX_OPERANDS];
    int64_t stride[MAX_OPERANDS][NK_MAX_RANK];
};

template <typename T, int NSRC, int FUNSET>
__global__ __launch_bounds__(256) void tile_kernel(TileArgs A, Prog P, T* __restrict__ drn, Ptrs srcs) {
    __shared__ T tile[64][65];
    const int last = A.rank - 1;
    const unsigned tx = threadIdx.x & 63, ty = threadIdx.x >> 6;   // 64 x 4
    for (unsigned blk = blockIdx.x; blk < A.n_blocks; blk += gridDim.x) {
        unsigned r = blk;
        unsigned q = A.div_tiles_l.div(r);
        const unsigned tl = r - q * A.tiles_l; r = q;
        q = A.div_tiles_p.div(r);
        const unsigned tp = r - q * A.tiles_p; r = q;
        int64_t off[NSRC + 1];
#pragma unroll
        for (int o = 0; o <= NSRC; o++) off[o] = A.base[o];
        for (int k = last - 1; k >= 0; k--) {
            if (k == A.pax) continue;
            const unsigned qq = A.outer[k].div(r);
            const unsigned idx = r - qq * A.outer[k].d;
            r = qq;
#pragma unroll
            for (int o = 0; o <= NSRC; o++) off[o] += (int64_t)idx * A.stride[o][k];
        }
        const unsigned p0 = tp * 64, l0 = tl * 64;
        T x[NSRC][16];
#pragma unroll
        for (int j = 0; j < NSRC; j++) {
            if (j < A.nsrc) {
                const T* sp = (const T*)srcs.p[j] + off[j + 1];
                const int64_t sP = A.stride[j + 1][A.pax], sL = A.stride[j + 1][last];
                if ((A.turned >> j) & 1u) {
                    __syncthreads();
#pragma unroll
                    for (int it = 0; it < 16; it++) {
                        const unsigned l = l0 + ty + 4 * it, p = p0 + tx;
                        if (l < A.L && p < A.P) tile[ty + 4 * it][tx] = sp[(int64_t)p * sP + (int64_t)l * sL];
                    }
                    __syncthreads();
#pragma unroll
                    for (int it = 0; it < 16; it++) x[j][it] = tile[tx][ty + 4 * it];
                } else {
#pragma unroll
                    for (int it = 0; it < 16; it++) {
                        const unsigned p = p0 + ty + 4 * it, l = l0 + tx;
                        x[j][it] = (p < A.P && l < A.L) ? sp[(int64_t)p * sP + (int64_t)l * sL] : T(0);
                    }
                }
            } else {
#pragma unroll
                for (int it = 0; it < 16; it++) x[j][it] = T(0);
            }
        }
        const int64_t dP = A.stride[0][A.pax], dL = A.stride[0][last];
        T out[16];
        run_prog<T, 16, NSRC, FUNSET>(P, x, out);
#pragma unroll
        for (int it = 0; it < 16; it++) {
            const unsigned p = p0 + ty + 4 * it, l = l0 + tx;
            if (p < A.P && l < A.L) {
                T* dst = drn + off[0] + (int64_t)p * dP + (int64_t)l * dL;
                if (A.streaming) __builtin_nontemporal_store(out[it], dst); else *dst = out[it];
            }
        }
    }
}

// ---- literal kernel: any descriptor, the reference's index formula --------------------------------------
// `own` bit j: source j unravels the flat index with its own indicesMap (binary elementwise,
// scalarization), otherwise it is addressed with the drain's nd-index (activation, broadcast).
// `pin[j]` bit k: index of source j pinned to 0 on axis k (forward broadcast).
struct LiteralArgs {
    int rank;
    int nsrc;
    unsigned n;
    unsigned own;
    unsigned pin[NK_FUSE_MAX_SRC];
    Cfg cfg[MAX_OPERANDS];
};

template <typename T>
__global__ __launch_bounds__(256) void literal_kernel(LiteralArgs A, Prog P, T* __restrict__ drn, Ptrs srcs) {
    const unsigned step = gridDim.x * blockDim.x;
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < A.n; i += step) {
        int nd[NK_MAX_RANK];
        nd_of_flat(A.cfg[0], A.rank, (int)i, nd);
        const int pd = phys_of_nd(A.cfg[0], A.rank, nd);
        T x[NK_FUSE_MAX_SRC][1];
        for (int j = 0; j < NK_FUSE_MAX_SRC; j++) {
            x[j][0] = T(0);
            if (j < A.nsrc) {
                int ps;
                if ((A.own >> j) & 1u) ps = phys_of_flat(A.cfg[j + 1], A.rank, (int)i);
                else {
                    int sn[NK_MAX_RANK];
                    for (int k = 0; k < A.rank; k++) sn[k] = ((A.pin[j] >> k) & 1u) ? 0 : nd[k];
                    ps = phys_of_nd(A.cfg[j + 1], A.rank, sn);
                }
                x[j][0] = ((const T*)srcs.p[j])[ps];
            }
        }
        T out[1];
        run_prog<T, 1, NK_FUSE_MAX_SRC, 2>(P, x, out);
        drn[pd] = out[0];
    }
}

// ---- launch plan (filled by the host analysis, executed by launch_family<T, FUNSET>) --------------------
enum PlanKind { PLAN_ROWS, PLAN_TILE, PLAN_CANON, PLAN_LITERAL };
struct Plan {
    PlanKind kind;
    bool vec;                  // rows: 16-byte vectors
    int nsrc;
    unsigned grid;
    RowsArgs rows;
    TileArgs tile;
    CanonArgs canon;
    LiteralArgs literal;
    Prog prog;
    void* drn;
    Ptrs srcs;
};

template <typename T, int FUNSET> int launch_family(Device* dev, const Plan& plan);

}  // namespace nk
