// Device side of the elementwise kernel family (activation, binary elementwise, scalarization, fill,
// forward broadcast, fused expressions): "drain[i] = program(sources at i)".
//
// The host (nk_eltwise.hip) compiles each operation to a small accumulator program and reduces the view
// descriptors to one of four access patterns; the kernels here are instantiated per
//   T        float | double
//   FUNSET   0: + - * / and copies only   1: + the cheap forward activations   2: the full table
//            3: the full table on the packed interpreter (at most 16 instructions, one saved intermediate, 3 sources):
//               every derivative and every heavy function of a program that short -- the backward launch of every
//               activation and operator, the derivatives of a fused chain, sin / cos / log10 / cbrt / softplus / pow /
//               modulo by themselves; set 2 keeps the long and deep programs and those with more sources
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
constexpr int HW_STACK = NK_FUSE_MAX_SAVED;

struct alignas(32) Prog {
    unsigned code[MAX_INSTR];      // op | arg << 8 | src << 16, what the device reads: eight words per scalar load
    int n;
    unsigned char op[MAX_INSTR];   // I_*                                            (the host's view of the same program)
    unsigned char arg[MAX_INSTR];  // fun id | binary op | (binary op)*2 + d
    unsigned char src[MAX_INSTR];  // k | SRC_CONST0 + k | SRC_POP
    double consts[NK_FUSE_MAX_CONST];
};
static_assert(MAX_INSTR % 8 == 0, "the interpreter fetches the program in blocks of eight words");

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
    // The program is fetched eight instruction words at a time with one wide scalar load and consumed from a shift
    // register; the next eight are requested before the current ones run.  (One byte-sized scalar load per field and
    // instruction made every interpreted instruction wait out a trip to the scalar cache: 1.0 ms for the twelve
    // instructions of the chain's derivative over 2^26 elements.)
    unsigned n0 = P.code[0], n1 = P.code[1], n2 = P.code[2], n3 = P.code[3], n4 = P.code[4], n5 = P.code[5], n6 = P.code[6], n7 = P.code[7];
    for (int base = 0; base < P.n; base += 8) {
      unsigned c0 = n0, c1 = n1, c2 = n2, c3 = n3, c4 = n4, c5 = n5, c6 = n6, c7 = n7;
      const int nb = base + 8 < MAX_INSTR ? base + 8 : 0;               // (past the end: any block, it is not run)
      n0 = P.code[nb]; n1 = P.code[nb + 1]; n2 = P.code[nb + 2]; n3 = P.code[nb + 3]; n4 = P.code[nb + 4]; n5 = P.code[nb + 5]; n6 = P.code[nb + 6]; n7 = P.code[nb + 7];
      const int here = P.n - base < 8 ? P.n - base : 8;
      for (int i = 0; i < here; i++) {
        const unsigned code = c0;
        c0 = c1; c1 = c2; c2 = c3; c3 = c4; c4 = c5; c5 = c6; c6 = c7;
        const int op = code & 0xff, arg = (code >> 8) & 0xff, s = (code >> 16) & 0xff;
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
}

// Short programs (at most LIGHT_INSTR instructions, LIGHT_CONST constants, no saved intermediates) are
// handed to the specialised families in packed form: all instruction words sit in one aligned block of
// the kernel arguments and are fetched with a single wide scalar load, then consumed from a shift
// register, so the interpreter never waits for memory between instructions.
// Set 3 (derivative programs) takes twice as many instructions and one saved intermediate: the derivative of a chain
// f(g(..)) by an inner operand is f'(g(..)) saved, times g' computed after it.
constexpr int LIGHT_INSTR = 8, LIGHT_INSTR_D = 16, LIGHT_CONST = 4;
struct alignas(64) LightProg {
    unsigned code[LIGHT_INSTR_D];  // op | arg << 8 | src << 16
    double consts[LIGHT_CONST];
    int n;
};

template <typename T, int V, int NSRC, int FUNSET>
__device__ __forceinline__ void run_light(const LightProg& P, const T (&src)[NSRC][V], T (&acc)[V]) {
    constexpr int FS = FUNSET == 3 ? 2 : FUNSET;         // set 3 carries the whole function and operator table
    constexpr bool DERIV = FUNSET == 3;
    unsigned c0 = P.code[0], c1 = P.code[1], c2 = P.code[2], c3 = P.code[3], c4 = P.code[4], c5 = P.code[5], c6 = P.code[6], c7 = P.code[7];
    unsigned c8 = 0, c9 = 0, c10 = 0, c11 = 0, c12 = 0, c13 = 0, c14 = 0, c15 = 0;
    if constexpr (DERIV) { c8 = P.code[8]; c9 = P.code[9]; c10 = P.code[10]; c11 = P.code[11]; c12 = P.code[12]; c13 = P.code[13]; c14 = P.code[14]; c15 = P.code[15]; }
    T k[LIGHT_CONST];
#pragma unroll
    for (int i = 0; i < LIGHT_CONST; i++) k[i] = (T)P.consts[i];
    T saved[DERIV ? V : 1];
#pragma unroll
    for (int v = 0; v < (DERIV ? V : 1); v++) saved[v] = T(0);
#pragma unroll
    for (int v = 0; v < V; v++) acc[v] = T(0);
    for (int pc = 0; pc < P.n; pc++) {
        const unsigned code = c0;
        c0 = c1; c1 = c2; c2 = c3; c3 = c4; c4 = c5; c5 = c6; c6 = c7;
        if constexpr (DERIV) { c7 = c8; c8 = c9; c9 = c10; c10 = c11; c11 = c12; c12 = c13; c13 = c14; c14 = c15; }
        const int op = code & 0xff, arg = (code >> 8) & 0xff, s = (code >> 16) & 0xff;
        T x[V];
        if (DERIV && op == I_PUSH) {
#pragma unroll
            for (int v = 0; v < (DERIV ? V : 1); v++) saved[v] = acc[v];
            continue;
        }
        if (op != I_FUN && op != I_DFUN) {
            if (DERIV && s == SRC_POP) {
#pragma unroll
                for (int v = 0; v < (DERIV ? V : 1); v++) x[v] = saved[v];
            } else if (s >= SRC_CONST0) {
                T c = k[0];
#pragma unroll
                for (int i = 1; i < LIGHT_CONST; i++) if (s == SRC_CONST0 + i) c = k[i];
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
                if constexpr (FUNSET >= 1) apply_fun<T, V, FS>(arg, acc);
                break;
            case I_DFUN:
                if constexpr (FUNSET == 3) apply_dfun<T, V>(arg, acc);
                break;
            case I_BIN: apply_bin<T, V, FS>(arg, acc, x); break;
            case I_RBIN:
                apply_bin<T, V, FS>(arg, x, acc);
#pragma unroll
                for (int v = 0; v < V; v++) acc[v] = x[v];
                break;
            case I_DBIN: apply_dbin<T, V, FS>(arg >> 1, arg & 1, acc, x); break;
            case I_RDBIN:
                apply_dbin<T, V, FS>(arg >> 1, arg & 1, x, acc);
#pragma unroll
                for (int v = 0; v < V; v++) acc[v] = x[v];
                break;
        }
    }
}

// family-independent entry: the full family interprets the long form, the others the packed form
template <typename T, int V, int NSRC, int FUNSET>
__device__ __forceinline__ void run_any(const Prog& P, const LightProg& LP, const T (&src)[NSRC][V], T (&acc)[V]) {
    if constexpr (FUNSET == 2) run_prog<T, V, NSRC, FUNSET>(P, src, acc);
    else run_light<T, V, NSRC, FUNSET>(LP, src, acc);
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

// Vector access types are only element-aligned: gfx950 global loads and stores of 2 or 4 dwords need
// dword alignment only, so views that start at an odd element (slices) still move 16 bytes per lane.
template <typename T, int V> struct VecOf { typedef T type __attribute__((ext_vector_type(V), aligned(sizeof(T)))); };
template <typename T> struct VecOf<T, 1> { typedef T type; };

// NT: the value is read once by the whole launch -- a non-temporal load keeps it from displacing
// lines that will be used again and is measurably faster for streams far larger than the caches.
template <typename T, int V, bool NT = false>
__device__ __forceinline__ void load_vec(T (&dst)[V], const T* p) {
    if constexpr (V == 1) dst[0] = NT ? __builtin_nontemporal_load(p) : *p;
    else {
        typedef typename VecOf<T, V>::type Vec;
        Vec v;
        if constexpr (NT) v = __builtin_nontemporal_load((const Vec*)p); else v = *(const Vec*)p;
#pragma unroll
        for (int i = 0; i < V; i++) dst[i] = v[i];
    }
}
// Plain stores.  Non-temporal stores were measured on these kernels (several units per block) and lose 5..8 %;
// they pay only together with one unit per block (rows_binary_lean_kernel).  Such a choice has to be made at compile
// time: a store that is non-temporal in one branch and plain in the other is merged into one plain store.
template <typename T, int V>
__device__ __forceinline__ void store_vec(T* p, const T (&src)[V]) {
    if constexpr (V == 1) *p = src[0];
    else {
        typename VecOf<T, V>::type v;
#pragma unroll
        for (int i = 0; i < V; i++) v[i] = src[i];
        *(typename VecOf<T, V>::type*)p = v;
    }
}

// ---- rows kernel -----------------------------------------------------------------------------------
// Every operand is contiguous (stride 1) or constant (stride 0) along the innermost collapsed axis.
// The work is cut into units of (256 >> tpr_log2 rows) x (tpr threads x V elements); a block owns PASSES
// units: consecutive ones, or (forward broadcast) the same column chunk of PASSES consecutive row groups, so
// that an operand which does not change along the rows is the same piece of memory in every pass.  A thread
// issues the loads of all its passes, runs the program once over all of them, then stores.  When a row spans at least a wavefront (tpr >= 64) the row index is wave-uniform:
// the nd-index arithmetic then runs on the scalar unit.  Element offsets are 32-bit (the host checks),
// at most ROWS_MAX_OUTER outer axes (more fall to the canon kernel; kernels take MAXO of them); the argument block is small and
// fixed-size so that it is fetched with a few wide scalar loads at kernel start.
constexpr int ROWS_MAX_OUTER = 5;
// The kernels resolve ROWS_FAST_OUTER outer axes unless instantiated for more: two further (unused) steps in the
// address arithmetic of every pass cost the broadcast of [1024,1,512] o [1,2048,512] five per cent.
constexpr int ROWS_FAST_OUTER = 3;
// units per block of rows_kernel: enough loads in flight to cover latency, few enough registers to keep
// several wavefronts per SIMD (three sources x 16 values already costs half the occupancy).  The fused chain
// tanh(sig(a)*b+c) on 2^26 elements: one pass 6.71, two 6.71, four 6.46 TB/s -- its 62 vector instructions per
// element (110 us of issue time in a 160 us launch), not the access pattern, hold it below the 7.2 TB/s a bare
// three-reads-one-write kernel reaches.
// (the full interpreter family keeps one pass: its V = 4 instantiation already holds 190 registers, two passes spill)
constexpr int rows_passes(int funset, int nsrc) { return funset == 2 ? 1 : funset == 3 ? 2 : (nsrc >= 3 ? 2 : 4); }
struct RowsArgs {
    int nouter;                // collapsed outer axes, 0..ROWS_MAX_OUTER
    int nsrc;
    unsigned L;                // innermost extent
    unsigned n_rows;           // product of the outer extents
    int tpr_log2;              // threads per row, log2
    unsigned chunks;           // column chunks per row
    unsigned row_groups;       // groups of (256 >> tpr_log2) rows
    int pass_rows;             // a block's passes walk down the rows (same chunk) instead of along the chunks
    unsigned const_last;       // bit j: source j has stride 0 along the innermost axis
    unsigned strided_last;     // bit j: source j has a stride other than 0 or 1 along the innermost axis (every n-th column)
    int simple_loads;          // every source register is filled by a plain vector load
    int vec;                   // elements per thread and pass (1 or 16 / sizeof(T))
    int ragged;                // L is not a multiple of vec: the last vector of a row is moved back to end with the row
    int nt_loads;              // every source element is read exactly once: the host picks the non-temporal-load variant
    FastDiv chunk_div;
    FastDiv outer[ROWS_MAX_OUTER];           // outer[0] is the innermost outer axis
    int base[MAX_OPERANDS];
    int stride[MAX_OPERANDS][ROWS_MAX_OUTER];
    int last_stride[MAX_OPERANDS];           // innermost stride of every operand (1 for the drain)
    // bit j: source j repeats along the innermost axis with period[j + 1] elements -- a short innermost axis (rows of
    // three: channels-last data and a per-channel operand) merged with the axis above it, along which the source was
    // pinned; its element at column c is the one at c mod period
    unsigned periodic_last;
    FastDiv period[MAX_OPERANDS];
    // Rows of fewer than 256 vectors whose vector count is no power of two would leave lanes idle (48 vectors per row:
    // 16 of 64): then the threads are numbered through all rows without gaps -- vector f of the launch is vector
    // f mod flat_vpr of row f / flat_vpr -- and `row_groups` counts units of 256 such vectors.  d == 1: not in use.
    FastDiv flat_vpr;
};

// addressing shared by the rows kernels: unit -> (row, col), row -> element offset of every operand
template <int NOPS>
struct RowsAddr {
    int off[NOPS];
    unsigned col;
    bool live;
};
template <int NOPS, int MAXO = ROWS_FAST_OUTER>
__device__ __forceinline__ RowsAddr<NOPS> rows_address(const RowsArgs& A, unsigned rg, unsigned chunk) {
    const unsigned tpr = 1u << A.tpr_log2;
    const unsigned rows_per_pass = 256u >> A.tpr_log2;
    const unsigned sub = threadIdx.x >> A.tpr_log2, lane = threadIdx.x & (tpr - 1);
    unsigned row = rg * rows_per_pass + sub;                        // rg and chunk are block-uniform
    RowsAddr<NOPS> R;
    R.col = (chunk * tpr + lane) * (unsigned)A.vec;
    if (A.flat_vpr.d > 1) {                                         // threads numbered through the rows without gaps
        const unsigned f = rg * 256u + threadIdx.x;
        row = A.flat_vpr.div(f);
        R.col = (f - row * A.flat_vpr.d) * (unsigned)A.vec;
    }
    const bool row_ok = rg < A.row_groups && row < A.n_rows;        // wave-uniform when a row spans a wavefront
    R.live = row_ok && R.col < A.L;
    if (!row_ok) row = 0;                                           // dead lanes get a valid address:
    if (!R.live) R.col = 0;                                         // loads need no predicate
    if (A.ragged && R.col + (unsigned)A.vec > A.L) R.col = A.L - (unsigned)A.vec;
    auto resolve = [&](unsigned r) {
#pragma unroll
        for (int o = 0; o < NOPS; o++) R.off[o] = A.base[o];
#pragma unroll
        for (int k = 0; k < MAXO; k++) {
            if (k < A.nouter) {
                const unsigned q = A.outer[k].div(r);
                const int idx = (int)(r - q * A.outer[k].d);
                r = q;
#pragma unroll
                for (int o = 0; o < NOPS; o++) R.off[o] += idx * A.stride[o][k];
            }
        }
    };
    // a row that spans a whole wavefront is wave-uniform: resolve it on the scalar unit
    if (A.tpr_log2 >= 6 && A.flat_vpr.d <= 1) resolve(__builtin_amdgcn_readfirstlane(row));
    else resolve(row);
    return R;
}

// (block id, pass) -> (row group, column chunk).  Units are numbered with the chunk varying fastest; a block
// either owns `passes` consecutive units, or -- pass_rows -- the same chunk of `passes` consecutive row groups.
__device__ __forceinline__ void rows_unit(const RowsArgs& A, int passes, int p, unsigned& rg, unsigned& chunk) {
    if (A.pass_rows) {
        const unsigned rgb = A.chunk_div.div(blockIdx.x);
        chunk = blockIdx.x - rgb * A.chunks;
        rg = rgb * (unsigned)passes + (unsigned)p;
    } else {
        const unsigned u = blockIdx.x * (unsigned)passes + (unsigned)p;
        rg = A.chunk_div.div(u);
        chunk = u - rg * A.chunks;
    }
}

template <typename T, int V, int NSRC, int FUNSET, int PASSES, bool NT = false, int MAXO = ROWS_FAST_OUTER>
__global__ __launch_bounds__(256) void rows_kernel(RowsArgs A, Prog P, LightProg LP, T* __restrict__ drn, Ptrs srcs) {
    T x[NSRC][PASSES * V];
    int doff[PASSES];
    bool live[PASSES];
    if (A.simple_loads) {
        // every source is a plain vector load: no branches between the loads of all passes
#pragma unroll
        for (int p = 0; p < PASSES; p++) {
            unsigned rg, chunk;
            rows_unit(A, PASSES, p, rg, chunk);
            const RowsAddr<NSRC + 1> R = rows_address<NSRC + 1, MAXO>(A, rg, chunk);
            live[p] = R.live;
            doff[p] = R.off[0] + (int)R.col;
#pragma unroll
            for (int j = 0; j < NSRC; j++) {
                T (&xj)[V] = *reinterpret_cast<T (*)[V]>(&x[j][p * V]);
                load_vec<T, V, NT>(xj, (const T*)srcs.p[j] + R.off[j + 1] + R.col);
            }
        }
    } else {
#pragma unroll
        for (int p = 0; p < PASSES; p++) {
            unsigned rg, chunk;
            rows_unit(A, PASSES, p, rg, chunk);
            const RowsAddr<NSRC + 1> R = rows_address<NSRC + 1, MAXO>(A, rg, chunk);
            live[p] = R.live;
            doff[p] = R.off[0] + (int)R.col;
#pragma unroll
            for (int j = 0; j < NSRC; j++) {
                T (&xj)[V] = *reinterpret_cast<T (*)[V]>(&x[j][p * V]);
                if (j < A.nsrc) {
                    const T* sp = (const T*)srcs.p[j] + R.off[j + 1];
                    if ((A.const_last >> j) & 1u) {
                        const T c = *sp;
#pragma unroll
                        for (int v = 0; v < V; v++) xj[v] = c;
                    } else if ((A.strided_last >> j) & 1u) {
                        const int ls = A.last_stride[j + 1];
#pragma unroll
                        for (int v = 0; v < V; v++) xj[v] = sp[(int)(R.col + v) * ls];
                    } else if ((A.periodic_last >> j) & 1u) {
                        const unsigned period = A.period[j + 1].d;
                        const unsigned first = R.col - A.period[j + 1].div(R.col) * period;      // col mod period
#pragma unroll
                        for (int v = 0; v < V; v++) {
                            unsigned at = first + v;                   // < period + 4: at most two periods too far
                            at = at >= period ? at - period : at;
                            at = at >= period ? at - period : at;
                            xj[v] = sp[at];                            // (loading the period once and selecting would make
                        }                                              // the passes wait for one another: measured slower)
                    } else {
                        load_vec<T, V>(xj, sp + R.col);
                    }
                } else {
#pragma unroll
                    for (int v = 0; v < V; v++) xj[v] = T(0);
                }
            }
        }
    }
    T out[PASSES * V];
    run_any<T, PASSES * V, NSRC, FUNSET>(P, LP, x, out);
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
        if (live[p]) {
            T (&op)[V] = *reinterpret_cast<T (*)[V]>(&out[p * V]);
            store_vec<T, V>(drn + doff[p], op);
        }
    }
}

// drain = f(src) or f'(src) for ONE function of the table, known at compile time: what nk_activation launches.  The data
// path is rows_kernel's (plain vector loads, two units per block); the function is inlined instead of interpreted, so a
// thread spends its instructions on the function alone.  That matters where the function, not memory, bounds the kernel:
// the f32 derivatives that repeat the reference's double-precision formula (tanh', 2^26 elements: 56 vector instructions
// per element and 0.49 of the HBM rate through the interpreter, 0.61-0.63 here) -- and the light functions lose nothing.
constexpr int SINGLE_PASSES = 2;
template <typename T, int V, bool NT, bool DERIV, int FID>
__global__ __launch_bounds__(256) void rows_single_kernel(RowsArgs A, T* __restrict__ drn, const T* __restrict__ src) {
    T x[SINGLE_PASSES * V];
    int doff[SINGLE_PASSES];
    bool live[SINGLE_PASSES];
#pragma unroll
    for (int p = 0; p < SINGLE_PASSES; p++) {
        unsigned rg, chunk;
        rows_unit(A, SINGLE_PASSES, p, rg, chunk);
        const RowsAddr<2> R = rows_address<2>(A, rg, chunk);
        live[p] = R.live;
        doff[p] = R.off[0] + (int)R.col;
        T (&xp)[V] = *reinterpret_cast<T (*)[V]>(&x[p * V]);
        load_vec<T, V, NT>(xp, src + R.off[1] + R.col);
    }
    if constexpr (DERIV) apply_dfun<T, SINGLE_PASSES * V, dfun_calls_library(FID)>(FID, x);
    else apply_fun<T, SINGLE_PASSES * V, (fun_is_heavy(FID) ? 2 : 1)>(FID, x);
#pragma unroll
    for (int p = 0; p < SINGLE_PASSES; p++) {
        if (live[p]) {
            T (&op)[V] = *reinterpret_cast<T (*)[V]>(&x[p * V]);
            store_vec<T, V>(drn + doff[p], op);
        }
    }
}

// drain = src0 op b, or a partial derivative of it, for ONE heavy operator known at compile time (modulo, power, and
// the derivatives of division, modulo and power -- the operators the four-operator kernel below does not carry); b is
// source 1 or a constant (scalarization).  Same data path as rows_single_kernel.
// KIND 0: the operator; 1, 2: its derivative by operand 0, 1.
template <typename T, int V, bool NT, int KIND, int OP, bool CONST_B>
__global__ __launch_bounds__(256) void rows_pair_kernel(RowsArgs A, T* __restrict__ drn, const T* __restrict__ s0, const T* __restrict__ s1, T k) {
    T x[SINGLE_PASSES * V], y[SINGLE_PASSES * V];
    int doff[SINGLE_PASSES];
    bool live[SINGLE_PASSES];
#pragma unroll
    for (int p = 0; p < SINGLE_PASSES; p++) {
        unsigned rg, chunk;
        rows_unit(A, SINGLE_PASSES, p, rg, chunk);
        const RowsAddr<3> R = rows_address<3>(A, rg, chunk);
        live[p] = R.live;
        doff[p] = R.off[0] + (int)R.col;
        T (&xp)[V] = *reinterpret_cast<T (*)[V]>(&x[p * V]);
        T (&yp)[V] = *reinterpret_cast<T (*)[V]>(&y[p * V]);
        load_vec<T, V, NT>(xp, s0 + R.off[1] + R.col);
        if constexpr (CONST_B) {
#pragma unroll
            for (int v = 0; v < V; v++) yp[v] = k;
        } else load_vec<T, V, NT>(yp, s1 + R.off[2] + R.col);
    }
    constexpr bool ONE = sizeof(T) == 8;       // the double-precision library routines: one element at a time (registers)
    if constexpr (KIND == 0) apply_bin<T, SINGLE_PASSES * V, 2, ONE>(OP, x, y);
    else apply_dbin<T, SINGLE_PASSES * V, 2, ONE>(OP, KIND - 1, x, y);
#pragma unroll
    for (int p = 0; p < SINGLE_PASSES; p++) {
        if (live[p]) {
            T (&op)[V] = *reinterpret_cast<T (*)[V]>(&x[p * V]);
            store_vec<T, V>(drn + doff[p], op);
        }
    }
}

// drain = src0 op src1 with op in {+, -, *, /} and plain aligned loads: the bandwidth-critical case
// (same-shape elementwise and forward broadcast).  The operator is resolved once, outside the passes,
// and each pass is stored as soon as its operands have arrived.
// HOIST bit j: source j does not change along the rows a block covers (forward broadcast): it is loaded once.
// CONST bit j: source j does not change along a row (one element per row, e.g. a per-row scale or an outer product).
// PERIODIC bit j: source j repeats along the row with a period shorter than a vector (RowsArgs::periodic_last): its
//                 elements are gathered at column mod period, all gathers of all passes requested before the first use.
template <typename T, int V, int PASSES, bool NT = false, int HOIST = 0, int CONST = 0, int MAXO = ROWS_FAST_OUTER, int PERIODIC = 0>
__global__ __launch_bounds__(256) void rows_binary_kernel(RowsArgs A, int op, T* __restrict__ drn, const T* __restrict__ s0,
                                                          const T* __restrict__ s1) {
    T x0[PASSES][V], x1[PASSES][V];
    int doff[PASSES];
    bool live[PASSES];
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
        unsigned rg, chunk;
        rows_unit(A, PASSES, p, rg, chunk);
        const RowsAddr<3> R = rows_address<3, MAXO>(A, rg, chunk);
        live[p] = R.live;
        doff[p] = R.off[0] + (int)R.col;
        auto gather = [&](T (&x)[V], const T* sp, int operand) {
            const unsigned period = A.period[operand].d;
            const unsigned first = R.col - A.period[operand].div(R.col) * period;          // col mod period
            _Pragma("unroll") for (int v = 0; v < V; v++) {
                unsigned at = first + v;                                                   // at most two periods too far
                at = at >= period ? at - period : at;
                at = at >= period ? at - period : at;
                x[v] = sp[at];
            }
        };
        if (PERIODIC & 1) gather(x0[p], s0 + R.off[1], 1);
        else if (CONST & 1) { const T c = s0[R.off[1]]; _Pragma("unroll") for (int v = 0; v < V; v++) x0[p][v] = c; }
        else if (p == 0 || !(HOIST & 1)) load_vec<T, V, NT>(x0[p], s0 + R.off[1] + R.col);
        if (PERIODIC & 2) gather(x1[p], s1 + R.off[2], 2);
        else if (CONST & 2) { const T c = s1[R.off[2]]; _Pragma("unroll") for (int v = 0; v < V; v++) x1[p][v] = c; }
        else if (p == 0 || !(HOIST & 2)) load_vec<T, V, NT>(x1[p], s1 + R.off[2] + R.col);
    }
    if (HOIST) {
#pragma unroll
        for (int p = 1; p < PASSES; p++)
#pragma unroll
            for (int v = 0; v < V; v++) {
                if (HOIST & 1) x0[p][v] = x0[0][v];
                if (HOIST & 2) x1[p][v] = x1[0][v];
            }
    }
#define NK_BINARY_PASSES(EXPR)                                                        \
    _Pragma("unroll") for (int p = 0; p < PASSES; p++) {                              \
        T out[V];                                                                     \
        _Pragma("unroll") for (int v = 0; v < V; v++) { const T a = x0[p][v], b = x1[p][v]; out[v] = (EXPR); } \
        if (live[p]) store_vec<T, V>(drn + doff[p], out);                                     \
    }
    switch (op) {
        case NK_OP_ADD: NK_BINARY_PASSES(a + b) break;
        case NK_OP_SUB: NK_BINARY_PASSES(a - b) break;
        case NK_OP_MUL: NK_BINARY_PASSES(a * b) break;
        default: NK_BINARY_PASSES(a / b) break;
    }
#undef NK_BINARY_PASSES
}

// Large outputs (the write stream dominates): one unit per block and non-temporal stores.  Measured with a plain
// fill of 4 GiB, blocks that write 4 KiB each in dispatch order reach 6.9 TB/s where blocks of 32 KiB reach 5.8: the
// window of memory that is being written at one time stays small and moves front to back.  Non-temporal stores
// keep the output from displacing the (re-used) sources in L2, so the short blocks' loads return quickly; the
// prologue is kept short for the same reason -- a compact argument block read at once, the number of outer axes a
// template parameter, rows resolved on the scalar unit.
struct LeanArgs {
    unsigned n_rows, L;
    int tpr_log2;              // threads per row, log2
    unsigned chunks;           // column chunks per row
    int op;
    int ragged;                // L is not a multiple of V: the last vector of a row is moved back to end with the row
    FastDiv chunk_div;
    FastDiv outer[ROWS_FAST_OUTER];          // outer[0] is the innermost outer axis
    int base[3];
    int stride[3][ROWS_FAST_OUTER];
    FastDiv flat_vpr;          // d > 1: threads numbered through the rows without gaps (RowsArgs::flat_vpr); the drain is dense,
                               // so every block still writes one contiguous, aligned unit whatever the row length
};
// CONST bit j: source j does not change along a row (one element per row).  WIDE: a row spans at least a wavefront, so
// its index is wave-uniform and is resolved on the scalar unit.
template <typename T, int V, int NOUT, int CONST, bool WIDE>
__global__ __launch_bounds__(256) void rows_binary_lean_kernel(LeanArgs A, T* __restrict__ drn, const T* __restrict__ s0, const T* __restrict__ s1) {
    const unsigned tpr = 1u << A.tpr_log2, rpp = 256u >> A.tpr_log2;
    const unsigned rg = A.chunk_div.div(blockIdx.x), chunk = blockIdx.x - rg * A.chunks;
    const unsigned sub = threadIdx.x >> A.tpr_log2, lane = threadIdx.x & (tpr - 1);
    unsigned row = rg * rpp + sub, col = (chunk * tpr + lane) * (unsigned)V;
    if (A.flat_vpr.d > 1) {
        const unsigned f = blockIdx.x * 256u + threadIdx.x;
        row = A.flat_vpr.div(f);
        col = (f - row * A.flat_vpr.d) * (unsigned)V;
    }
    const bool row_ok = row < A.n_rows;
    const bool live = row_ok && col < A.L;
    if (!row_ok) row = 0;                        // dead lanes get a valid address: the loads need no predicate
    if (!live) col = 0;
    if (A.ragged && col + (unsigned)V > A.L) col = A.L - (unsigned)V;
    unsigned r = WIDE ? (unsigned)__builtin_amdgcn_readfirstlane(row) : row;
    int off0 = A.base[0], off1 = A.base[1], off2 = A.base[2];
#pragma unroll
    for (int k = 0; k < NOUT; k++) {
        const unsigned q = A.outer[k].div(r);
        const int idx = (int)(r - q * A.outer[k].d);
        r = q;
        off0 += idx * A.stride[0][k]; off1 += idx * A.stride[1][k]; off2 += idx * A.stride[2][k];
    }
    T a[V], b[V], out[V];
    if constexpr (CONST & 1) { const T c = s0[off1]; _Pragma("unroll") for (int v = 0; v < V; v++) a[v] = c; }
    else load_vec<T, V>(a, s0 + off1 + col);
    if constexpr (CONST & 2) { const T c = s1[off2]; _Pragma("unroll") for (int v = 0; v < V; v++) b[v] = c; }
    else load_vec<T, V>(b, s1 + off2 + col);
    switch (A.op) {
        case NK_OP_ADD: _Pragma("unroll") for (int v = 0; v < V; v++) out[v] = a[v] + b[v]; break;
        case NK_OP_SUB: _Pragma("unroll") for (int v = 0; v < V; v++) out[v] = a[v] - b[v]; break;
        case NK_OP_MUL: _Pragma("unroll") for (int v = 0; v < V; v++) out[v] = a[v] * b[v]; break;
        default:        _Pragma("unroll") for (int v = 0; v < V; v++) out[v] = a[v] / b[v]; break;
    }
    if (live) {
        typename VecOf<T, V>::type w;
#pragma unroll
        for (int v = 0; v < V; v++) w[v] = out[v];
        __builtin_nontemporal_store(w, (typename VecOf<T, V>::type*)(drn + off0 + col));
    }
}

// drain = one value, large outputs: the same layout without sources (plain stores: with nothing to keep in L2 they
// are the faster ones, 6.9 against 6.7 TB/s)
template <typename T, int V, int NOUT, bool WIDE>
__global__ __launch_bounds__(256) void rows_fill_lean_kernel(LeanArgs A, T value, T* __restrict__ drn) {
    const unsigned tpr = 1u << A.tpr_log2, rpp = 256u >> A.tpr_log2;
    const unsigned rg = A.chunk_div.div(blockIdx.x), chunk = blockIdx.x - rg * A.chunks;
    const unsigned sub = threadIdx.x >> A.tpr_log2, lane = threadIdx.x & (tpr - 1);
    const unsigned row = rg * rpp + sub;
    unsigned col = (chunk * tpr + lane) * (unsigned)V;
    if (row >= A.n_rows || col >= A.L) return;
    if (A.ragged && col + (unsigned)V > A.L) col = A.L - (unsigned)V;
    unsigned r = WIDE ? (unsigned)__builtin_amdgcn_readfirstlane(row) : row;
    int off0 = A.base[0];
#pragma unroll
    for (int k = 0; k < NOUT; k++) {
        const unsigned q = A.outer[k].div(r);
        off0 += (int)(r - q * A.outer[k].d) * A.stride[0][k];
        r = q;
    }
    T out[V];
#pragma unroll
    for (int v = 0; v < V; v++) out[v] = value;
    store_vec<T, V>(drn + off0 + col, out);
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
__global__ __launch_bounds__(256) void canon_kernel(CanonArgs A, Prog P, LightProg LP, T* __restrict__ drn, Ptrs srcs) {
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
        run_any<T, 1, NSRC, FUNSET>(P, LP, x, out);
        drn[off[0]] = out[0];
    }
}

// ---- tile_transpose kernel ----------------------------------------------------------------------------
// Collapsed axis `pax` (not the innermost) is the contiguous one of the sources flagged in `turned`; all
// other operands are contiguous or constant along the innermost axis.  A block owns a TILE_P (pax) x
// TILE_L (innermost) tile for one combination of the remaining axes.  Turned sources are read with 16-byte
// accesses along pax into one padded LDS tile each (all loads in flight before the single barrier) and
// handed to the lanes that own 16-byte pieces along the innermost axis; the drain is written with
// 16-byte stores.  64 x 32 keeps a thread at 8 elements per source and a block at 25 KB of LDS (f32), so
// that several blocks share a compute unit; measured on this part, longer runs on the read side matter
// more than on the write side.
constexpr int TILE_P = 64, TILE_L = 32;
struct TileArgs {
    int rank;
    int nsrc;
    int pax;
    unsigned turned;                        // bit j: source j is read along pax
    unsigned P, L;                          // extents of pax and of the innermost axis
    unsigned tiles_p, tiles_l;
    unsigned n_blocks;
    int group_log2, group_p_log2;           // blocks are numbered through groups of (1 << group_p_log2) x (1 << group_log2) tiles
    int nt_loads;                           // every source element is read exactly once: the host picks the non-temporal-load variant
    int careful;                            // some direct operand is constant along the innermost axis: no vector path
    int xcd_regions;                        // XCD x (blocks x, x + 8, ...) takes the x-th eighth of the tile order
    FastDiv div_tiles_l, div_tiles_p;
    FastDiv outer[NK_MAX_RANK];             // extents of the remaining axes
    int64_t base[MAX_OPERANDS];
    int64_t stride[MAX_OPERANDS][NK_MAX_RANK];
};

template <typename T, int NSRC, int FUNSET, bool NT = false>
__global__ __launch_bounds__(256) void tile_kernel(TileArgs A, Prog P, LightProg LP, T* __restrict__ drn, Ptrs srcs) {
    constexpr int VEC = 16 / sizeof(T);            // elements per 16-byte access
    constexpr int EPT = TILE_P * TILE_L / 256;     // elements per thread and operand (8)
    // read side: 16-byte pieces along pax
    constexpr int R_LPR = TILE_P / VEC;            // lanes that cover one tile row of a turned source
    constexpr int R_RPI = 256 / R_LPR;             // tile rows covered by one access of the whole block
    constexpr int R_NIT = TILE_L / R_RPI;          // accesses per thread and turned source
    // write side (and direct sources): 16-byte pieces along the innermost axis
    constexpr int W_LPR = TILE_L / VEC;
    constexpr int W_RPI = 256 / W_LPR;
    constexpr int W_NIT = TILE_P / W_RPI;
    static_assert(R_NIT * VEC == EPT && W_NIT * VEC == EPT, "tile shape and block size disagree");
    __shared__ T tiles[NSRC][TILE_L][TILE_P + 1];
    const int last = A.rank - 1;

    // Blocks that run at the same time behind one L2 should be neighbours: the hardware deals consecutive block ids
    // round-robin to the 8 XCDs, so XCD x (blocks x, x + 8, ...) takes the x-th eighth of the tile order, and that
    // order runs through groups of GP x GL tiles -- the pieces one L2 reads (along pax) and writes (along the
    // innermost axis) at a time then add up to long contiguous runs on both sides.
    unsigned rest = blockIdx.x;
    if (A.xcd_regions) rest = (blockIdx.x & 7u) * (A.n_blocks >> 3) + (blockIdx.x >> 3);
    const unsigned GL = 1u << A.group_log2, GP = 1u << A.group_p_log2;
    const unsigned local = rest & (GL * GP - 1);
    rest >>= A.group_log2 + A.group_p_log2;
    unsigned d = A.div_tiles_l.div(rest);                  // divisors are the group counts tiles_l / GL and tiles_p / GP
    const unsigned tl = (rest - d * A.div_tiles_l.d) * GL + (local & (GL - 1)); rest = d;
    d = A.div_tiles_p.div(rest);
    const unsigned tp = (rest - d * A.div_tiles_p.d) * GP + (local >> A.group_log2); rest = d;
    int64_t off[NSRC + 1];
#pragma unroll
    for (int o = 0; o <= NSRC; o++) off[o] = A.base[o];
    for (int k = last - 1; k >= 0; k--) {
        if (k == A.pax) continue;
        const unsigned qq = A.outer[k].div(rest);
        const unsigned idx = rest - qq * A.outer[k].d;
        rest = qq;
#pragma unroll
        for (int o = 0; o <= NSRC; o++) off[o] += (int64_t)idx * A.stride[o][k];
    }
    const unsigned p0 = tp * TILE_P, l0 = tl * TILE_L;
    const int64_t dP = A.stride[0][A.pax];
    T x[NSRC][EPT];
    T out[EPT];

    // whole tile inside the tensor, every operand either along pax or along the innermost axis:
    // 16-byte accesses on both sides, one barrier
    if (p0 + TILE_P <= A.P && l0 + TILE_L <= A.L && !A.careful) {
        // Which 16-byte piece of a turned source a lane reads.  The four elements of a piece stay in one LDS row
        // (tiles[row][pax]), and the 32 lanes that write together should hit 32 different banks.
        // With 16 lanes side by side in one row (banks 4 * rq + e, rq = 0..15) lanes rq and rq + 8 collide; eight
        // lanes per row and four rows (row pitch 65: banks 4 * q + row + e) do not.  A wavefront still reads four
        // whole 256-byte rows per access, only the order of its lanes differs.
        unsigned rq = threadIdx.x % R_LPR, rr = threadIdx.x / R_LPR;
        if constexpr (R_LPR == 16 && sizeof(T) == 4) {
            rq = ((threadIdx.x >> 5) & 1u) * 8u + (threadIdx.x & 7u);
            rr = (threadIdx.x >> 6) * 4u + ((threadIdx.x >> 3) & 3u);
        }
        const unsigned wq = threadIdx.x % W_LPR, wr = threadIdx.x / W_LPR;
#pragma unroll
        for (int j = 0; j < NSRC; j++) {
            if (j < A.nsrc) {
                if ((A.turned >> j) & 1u) {
                    const T* sp = (const T*)srcs.p[j] + off[j + 1] + p0 + rq * VEC;      // stride 1 along pax
                    const int64_t sL = A.stride[j + 1][last];
#pragma unroll
                    for (int it = 0; it < R_NIT; it++) {
                        const unsigned ll = rr + R_RPI * it;
                        T v[VEC];
                        load_vec<T, VEC, NT>(v, sp + (int64_t)(l0 + ll) * sL);
#pragma unroll
                        for (int e = 0; e < VEC; e++) tiles[j][ll][rq * VEC + e] = v[e];
                    }
                } else {
                    const T* sp = (const T*)srcs.p[j] + off[j + 1] + l0 + wq * VEC;      // stride 1 along the innermost axis
                    const int64_t sP = A.stride[j + 1][A.pax];
#pragma unroll
                    for (int it = 0; it < W_NIT; it++) {
                        T (&xv)[VEC] = *reinterpret_cast<T (*)[VEC]>(&x[j][it * VEC]);
                        load_vec<T, VEC, NT>(xv, sp + (int64_t)(p0 + wr + W_RPI * it) * sP);
                    }
                }
            } else {
#pragma unroll
                for (int e = 0; e < EPT; e++) x[j][e] = T(0);
            }
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < NSRC; j++) {
            if (j < A.nsrc && ((A.turned >> j) & 1u)) {
#pragma unroll
                for (int it = 0; it < W_NIT; it++)
#pragma unroll
                    for (int e = 0; e < VEC; e++) x[j][it * VEC + e] = tiles[j][wq * VEC + e][wr + W_RPI * it];
            }
        }
        run_any<T, EPT, NSRC, FUNSET>(P, LP, x, out);
        T* dp = drn + off[0] + l0 + wq * VEC;
#pragma unroll
        for (int it = 0; it < W_NIT; it++) {
            T (&ov)[VEC] = *reinterpret_cast<T (*)[VEC]>(&out[it * VEC]);
            store_vec<T, VEC>(dp + (int64_t)(p0 + wr + W_RPI * it) * dP, ov);
        }
        return;
    }

    // edge tiles and operands that are constant along the innermost axis: element by element, bounds checked
    constexpr int S_RPI = 256 / TILE_P;            // rows of TILE_P lanes in the block
    const unsigned tx = threadIdx.x % TILE_P, ty = threadIdx.x / TILE_P;
#pragma unroll
    for (int j = 0; j < NSRC; j++) {
        if (j < A.nsrc && ((A.turned >> j) & 1u)) {
            const T* sp = (const T*)srcs.p[j] + off[j + 1];
            const int64_t sP = A.stride[j + 1][A.pax], sL = A.stride[j + 1][last];
            for (int it = 0; it < EPT; it++) {
                const unsigned l = l0 + ty + S_RPI * it, p = p0 + tx;
                if (l < A.L && p < A.P) tiles[j][ty + S_RPI * it][tx] = sp[(int64_t)p * sP + (int64_t)l * sL];
            }
        }
    }
    __syncthreads();
    // drain side of the slow path: lane -> innermost index, TILE_L lanes per row of the tile
    constexpr int D_RPI = 256 / TILE_L;
    const unsigned dx = threadIdx.x % TILE_L, dy = threadIdx.x / TILE_L;
#pragma unroll
    for (int j = 0; j < NSRC; j++) {
        if (j < A.nsrc) {
            if ((A.turned >> j) & 1u) {
#pragma unroll
                for (int it = 0; it < EPT; it++) x[j][it] = tiles[j][dx][dy + D_RPI * it];
            } else {
                const T* sp = (const T*)srcs.p[j] + off[j + 1];
                const int64_t sP = A.stride[j + 1][A.pax], sL = A.stride[j + 1][last];
#pragma unroll
                for (int it = 0; it < EPT; it++) {
                    const unsigned p = p0 + dy + D_RPI * it, l = l0 + dx;
                    x[j][it] = (p < A.P && l < A.L) ? sp[(int64_t)p * sP + (int64_t)l * sL] : T(0);
                }
            }
        } else {
#pragma unroll
            for (int it = 0; it < EPT; it++) x[j][it] = T(0);
        }
    }
    run_any<T, EPT, NSRC, FUNSET>(P, LP, x, out);
#pragma unroll
    for (int it = 0; it < EPT; it++) {
        const unsigned p = p0 + dy + D_RPI * it, l = l0 + dx;
        if (p < A.P && l < A.L) {
            T* dst = drn + off[0] + (int64_t)p * dP + l;
            *dst = out[it];
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
enum PlanKind { PLAN_ROWS, PLAN_ROWS_BINARY, PLAN_TILE, PLAN_CANON, PLAN_LITERAL };
struct Plan {
    PlanKind kind;
    bool vec;                  // rows: 16-byte vectors
    int hoist = 0;             // rows_binary_kernel: bit j = source j is loaded once per block
    int binary_op;             // PLAN_ROWS_BINARY
    int passes;                // PLAN_ROWS_BINARY: units per block (2, 4 or 8)
    bool lean = false;         // PLAN_ROWS_BINARY: rows_binary_lean_kernel (one unit per block, non-temporal stores)
    bool lean_fill = false;    // PLAN_ROWS: rows_fill_lean_kernel (the program is one constant)
    bool single = false;       // PLAN_ROWS: rows_single_kernel (the program is one function, or one derivative, of source 0)
    bool single_deriv = false;
    int single_fun = 0;
    int pair_kind = -1;        // PLAN_ROWS: rows_pair_kernel (one heavy operator of source 0 and source 1 or a constant): 0 the
    int pair_op = 0;           // operator, 1 / 2 its derivative by operand 0 / 1
    bool pair_const = false;
    double pair_value = 0;
    double fill_value = 0;
    int nsrc;
    unsigned grid;
    RowsArgs rows;
    TileArgs tile;
    CanonArgs canon;
    LiteralArgs literal;
    Prog prog;
    LightProg light;
    void* drn;
    Ptrs srcs;
};

template <typename T, int FUNSET> int launch_family(Device* dev, const Plan& plan);
template <typename T> int launch_single(Device* dev, const Plan& plan);

}  // namespace nk
