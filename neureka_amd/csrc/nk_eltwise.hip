// The elementwise kernel family: activation, binary elementwise, scalarization, fill, forward
// broadcast and fused expressions.  All of them are "drain[i] = program(sources at i)" and share one
// engine: the host compiles the operation to a tiny accumulator program, analyses the view
// descriptors and picks one of four kernels
//   rows            every operand is contiguous (or constant) along the innermost collapsed axis:
//                   coalesced 16-byte accesses, outer axes resolved once per row
//   tile_transpose  some source is contiguous along a different axis than the drain (permuted
//                   views): 64x64 tiles are turned through LDS so both sides stay coalesced
//   canon           any other strided combination: one element per thread, mul-shift divisions
//   literal         descriptors that do not reduce to base+strides: the reference's index formula
#include "nk_internal.h"
#include "nk_scalar.h"

namespace nk {

// ------------------------------------------------------------------------------------------------
// accumulator programs
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

struct ProgBuilder {
    Prog p{};
    bool ok = true;
    void emit(int op, int arg, int src) {
        if (p.n >= MAX_INSTR) { ok = false; return; }
        p.op[p.n] = (unsigned char)op; p.arg[p.n] = (unsigned char)arg; p.src[p.n] = (unsigned char)src;
        p.n++;
    }
};

// postfix (the public encoding of nk_fused) -> accumulator form
static int compile_postfix(Prog& out, const int32_t* program, int n_ops, const double* consts, int n_consts, int n_src) {
    enum { LAZY, ACC, SAVED };
    struct Entry { int kind; int src; };
    Entry st[NK_FUSE_MAX_STACK];
    int sp = 0, saved = 0;
    ProgBuilder b;
    for (int k = 0; k < n_consts; k++) b.p.consts[k] = consts[k];
    auto save_acc = [&]() {   // an ACC entry below the top must move to the hardware stack
        for (int i = 0; i < sp; i++)
            if (st[i].kind == ACC) { b.emit(I_PUSH, 0, 0); st[i].kind = SAVED; saved++; }
    };
    for (int t = 0; t < n_ops; t++) {
        int code = program[2 * t], arg = program[2 * t + 1];
        switch (code) {
            case NK_FUSE_LOAD:
                NK_REQUIRE(arg >= 0 && arg < n_src, "nk_fused: op %d loads source %d of %d", t, arg, n_src);
                NK_REQUIRE(sp < NK_FUSE_MAX_STACK, "nk_fused: stack deeper than %d at op %d", NK_FUSE_MAX_STACK, t);
                st[sp++] = {LAZY, arg};
                break;
            case NK_FUSE_CONST:
                NK_REQUIRE(arg >= 0 && arg < n_consts, "nk_fused: op %d uses constant %d of %d", t, arg, n_consts);
                NK_REQUIRE(sp < NK_FUSE_MAX_STACK, "nk_fused: stack deeper than %d at op %d", NK_FUSE_MAX_STACK, t);
                st[sp++] = {LAZY, SRC_CONST0 + arg};
                break;
            case NK_FUSE_FUN:
            case NK_FUSE_DFUN:
                NK_REQUIRE(arg >= 0 && arg < NK_FUN_COUNT, "nk_fused: op %d: unknown function id %d", t, arg);
                NK_REQUIRE(sp >= 1, "nk_fused: op %d applies a function to an empty stack", t);
                if (st[sp - 1].kind == LAZY) {
                    save_acc();
                    b.emit(I_SET, 0, st[sp - 1].src);
                    st[sp - 1].kind = ACC;
                }
                b.emit(code == NK_FUSE_FUN ? I_FUN : I_DFUN, arg, 0);
                break;
            case NK_FUSE_BIN: {
                NK_REQUIRE(arg >= NK_OP_ADD && arg <= NK_OP_POW, "nk_fused: op %d: unknown operator id %d", t, arg);
                NK_REQUIRE(sp >= 2, "nk_fused: op %d needs two operands, stack holds %d", t, sp);
                Entry rhs = st[sp - 1], lhs = st[sp - 2];
                sp -= 2;
                if (lhs.kind == ACC && rhs.kind == LAZY) b.emit(I_BIN, arg, rhs.src);
                else if (lhs.kind == LAZY && rhs.kind == ACC) b.emit(I_RBIN, arg, lhs.src);
                else if (lhs.kind == LAZY && rhs.kind == LAZY) {
                    save_acc();
                    b.emit(I_SET, 0, lhs.src);
                    b.emit(I_BIN, arg, rhs.src);
                } else if (lhs.kind == SAVED && rhs.kind == ACC) {
                    b.emit(I_RBIN, arg, SRC_POP);
                    saved--;
                } else
                    return set_error(NK_ERR_ARG, "nk_fused: op %d: malformed program", t);
                st[sp++] = {ACC, 0};
                break;
            }
            default:
                return set_error(NK_ERR_ARG, "nk_fused: op %d: unknown op-code %d", t, code);
        }
        NK_REQUIRE(saved <= HW_STACK, "nk_fused: expression needs more than %d saved intermediates", HW_STACK);
    }
    NK_REQUIRE(sp == 1, "nk_fused: program leaves %d values on the stack, expected 1", sp);
    if (st[0].kind == LAZY) b.emit(I_SET, 0, st[0].src);
    NK_REQUIRE(b.ok, "nk_fused: program too long");
    out = b.p;
    return NK_OK;
}

// ------------------------------------------------------------------------------------------------
// interpreter: V elements per thread; all control flow is uniform over the grid (it only depends on
// kernel arguments), so it costs scalar branches, not divergence.
template <typename T, int V>
__device__ __forceinline__ void run_prog(const Prog& P, const T (&src)[NK_FUSE_MAX_SRC][V], T (&acc)[V]) {
    T s0[V], s1[V], s2[V], s3[V];
#pragma unroll
    for (int v = 0; v < V; v++) { acc[v] = T(0); s0[v] = s1[v] = s2[v] = s3[v] = T(0); }
    for (int pc = 0; pc < P.n; pc++) {
        const int op = P.op[pc], arg = P.arg[pc], s = P.src[pc];
        T x[V];
        if (op == I_PUSH) {
#pragma unroll
            for (int v = 0; v < V; v++) { s3[v] = s2[v]; s2[v] = s1[v]; s1[v] = s0[v]; s0[v] = acc[v]; }
            continue;
        }
        if (op != I_FUN && op != I_DFUN) {
            if (s == SRC_POP) {
#pragma unroll
                for (int v = 0; v < V; v++) { x[v] = s0[v]; s0[v] = s1[v]; s1[v] = s2[v]; s2[v] = s3[v]; }
            } else if (s >= SRC_CONST0) {
                T c = (T)P.consts[s - SRC_CONST0];
#pragma unroll
                for (int v = 0; v < V; v++) x[v] = c;
            } else {
#pragma unroll
                for (int v = 0; v < V; v++) x[v] = src[0][v];
#pragma unroll
                for (int j = 1; j < NK_FUSE_MAX_SRC; j++)
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
            case I_FUN: apply_fun<T, V>(arg, acc); break;
            case I_DFUN: apply_dfun<T, V>(arg, acc); break;
            case I_BIN: apply_bin<T, V>(arg, acc, x); break;
            case I_RBIN:
                apply_bin<T, V>(arg, x, acc);
#pragma unroll
                for (int v = 0; v < V; v++) acc[v] = x[v];
                break;
            case I_DBIN: apply_dbin<T, V>(arg >> 1, arg & 1, acc, x); break;
            case I_RDBIN:
                apply_dbin<T, V>(arg >> 1, arg & 1, x, acc);
#pragma unroll
                for (int v = 0; v < V; v++) acc[v] = x[v];
                break;
        }
    }
}

// ------------------------------------------------------------------------------------------------
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

template <typename T, int V> struct alignas(sizeof(T) * V) Pack { T v[V]; };

// ------------------------------------------------------------------------------------------------
// rows kernel
struct RowsArgs {
    int rank;                  // collapsed rank >= 1
    int nsrc;
    unsigned L;                // innermost extent
    unsigned n_rows;           // product of the outer extents
    int tpr_log2;              // threads per row, log2
    int passes;                // rows handled by one thread per tile
    unsigned chunks;           // column chunks per row
    unsigned n_tiles;
    FastDiv chunk_div;
    FastDiv outer[NK_MAX_RANK];             // outer[k] divides by shape[k], k < rank-1
    int64_t base[MAX_OPERANDS];
    int64_t stride[MAX_OPERANDS][NK_MAX_RANK];
};

template <typename T, int V>
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
        for (int p = 0; p < A.passes; p++) {
            const unsigned row = (row_tile * A.passes + p) * rows_per_pass + sub;
            if (row >= A.n_rows) break;
            int64_t off[MAX_OPERANDS];
#pragma unroll
            for (int o = 0; o < MAX_OPERANDS; o++) off[o] = A.base[o];
            unsigned r = row;
            for (int k = last - 1; k >= 0; k--) {
                unsigned q = A.outer[k].div(r);
                unsigned idx = r - q * A.outer[k].d;
                r = q;
#pragma unroll
                for (int o = 0; o < MAX_OPERANDS; o++)
                    if (o <= A.nsrc) off[o] += (int64_t)idx * A.stride[o][k];
            }
            T x[NK_FUSE_MAX_SRC][V];
#pragma unroll
            for (int j = 0; j < NK_FUSE_MAX_SRC; j++) {
                if (j < A.nsrc) {
                    const T* sp = (const T*)srcs.p[j] + off[j + 1];
                    if (A.stride[j + 1][last] != 0) {
                        Pack<T, V> pk = *(const Pack<T, V>*)(sp + col);
#pragma unroll
                        for (int v = 0; v < V; v++) x[j][v] = pk.v[v];
                    } else {
                        T c = *sp;
#pragma unroll
                        for (int v = 0; v < V; v++) x[j][v] = c;
                    }
                } else {
#pragma unroll
                    for (int v = 0; v < V; v++) x[j][v] = T(0);
                }
            }
            Pack<T, V> out;
            run_prog<T, V>(P, x, out.v);
            *(Pack<T, V>*)(drn + off[0] + col) = out;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// canon kernel: arbitrary strides, one element per thread
struct CanonArgs {
    int rank;
    int nsrc;
    unsigned n;
    FastDiv dims[NK_MAX_RANK];
    int64_t base[MAX_OPERANDS];
    int64_t stride[MAX_OPERANDS][NK_MAX_RANK];
};

template <typename T>
__global__ __launch_bounds__(256) void canon_kernel(CanonArgs A, Prog P, T* __restrict__ drn, Ptrs srcs) {
    const unsigned step = gridDim.x * blockDim.x;
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < A.n; i += step) {
        int64_t off[MAX_OPERANDS];
#pragma unroll
        for (int o = 0; o < MAX_OPERANDS; o++) off[o] = A.base[o];
        unsigned r = i;
        for (int k = A.rank - 1; k >= 0; k--) {
            unsigned q = A.dims[k].div(r);
            unsigned idx = r - q * A.dims[k].d;
            r = q;
#pragma unroll
            for (int o = 0; o < MAX_OPERANDS; o++)
                if (o <= A.nsrc) off[o] += (int64_t)idx * A.stride[o][k];
        }
        T x[NK_FUSE_MAX_SRC][1];
#pragma unroll
        for (int j = 0; j < NK_FUSE_MAX_SRC; j++) x[j][0] = j < A.nsrc ? ((const T*)srcs.p[j])[off[j + 1]] : T(0);
        T out[1];
        run_prog<T, 1>(P, x, out);
        drn[off[0]] = out[0];
    }
}

// ------------------------------------------------------------------------------------------------
// tile_transpose kernel.  Collapsed axis `pax` (not the innermost) is the contiguous one of the
// sources flagged in `turned`; all other operands are contiguous or constant along the innermost
// axis.  A block owns a 64 (pax) x 64 (innermost) tile for one combination of the remaining axes.
struct TileArgs {
    int rank;
    int nsrc;
    int pax;
    unsigned turned;                        // bit j: source j is read along pax
    unsigned P, L;                          // extents of pax and of the innermost axis
    unsigned tiles_p, tiles_l;
    unsigned n_blocks;
    FastDiv div_tiles_l, div_tiles_p;
    FastDiv outer[NK_MAX_RANK];             // extents of the remaining axes
    int64_t base[MAX_OPERANDS];
    int64_t stride[MAX_OPERANDS][NK_MAX_RANK];
};

template <typename T>
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
        int64_t off[MAX_OPERANDS];
#pragma unroll
        for (int o = 0; o < MAX_OPERANDS; o++) off[o] = A.base[o];
        for (int k = last - 1; k >= 0; k--) {
            if (k == A.pax) continue;
            unsigned qq = A.outer[k].div(r);
            unsigned idx = r - qq * A.outer[k].d;
            r = qq;
#pragma unroll
            for (int o = 0; o < MAX_OPERANDS; o++)
                if (o <= A.nsrc) off[o] += (int64_t)idx * A.stride[o][k];
        }
        const unsigned p0 = tp * 64, l0 = tl * 64;
        T x[NK_FUSE_MAX_SRC][16];
#pragma unroll
        for (int j = 0; j < NK_FUSE_MAX_SRC; j++) {
            if (j < A.nsrc) {
                const T* sp = (const T*)srcs.p[j] + off[j + 1];
                const int64_t sP = A.stride[j + 1][A.pax], sL = A.stride[j + 1][last];
                if ((A.turned >> j) & 1u) {
                    __syncthreads();
                    // read with tx along pax (stride 1 for this source)
#pragma unroll
                    for (int it = 0; it < 16; it++) {
                        unsigned l = l0 + ty + 4 * it, p = p0 + tx;
                        if (l < A.L && p < A.P) tile[ty + 4 * it][tx] = sp[(int64_t)p * sP + (int64_t)l * sL];
                    }
                    __syncthreads();
#pragma unroll
                    for (int it = 0; it < 16; it++) x[j][it] = tile[tx][ty + 4 * it];
                } else {
#pragma unroll
                    for (int it = 0; it < 16; it++) {
                        unsigned p = p0 + ty + 4 * it, l = l0 + tx;
                        x[j][it] = (p < A.P && l < A.L) ? sp[(int64_t)p * sP + (int64_t)l * sL] : T(0);
                    }
                }
            } else {
#pragma unroll
                for (int it = 0; it < 16; it++) x[j][it] = T(0);
            }
        }
        T out[16];
        run_prog<T, 16>(P, x, out);
        const int64_t dP = A.stride[0][A.pax], dL = A.stride[0][last];
#pragma unroll
        for (int it = 0; it < 16; it++) {
            unsigned p = p0 + ty + 4 * it, l = l0 + tx;
            if (p < A.P && l < A.L) drn[off[0] + (int64_t)p * dP + (int64_t)l * dL] = out[it];
        }
    }
}

// ------------------------------------------------------------------------------------------------
// literal kernel: any descriptor, the reference's formula.  `own` bit j: source j unravels the flat
// index with its own indicesMap (binary elementwise, scalarization), otherwise it is addressed with
// the drain's nd-index (activation, broadcast).  `pin[j]` bit k: index of source j pinned to 0 on
// axis k (forward broadcast).
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
        run_prog<T, 1>(P, x, out);
        drn[pd] = out[0];
    }
}

// ------------------------------------------------------------------------------------------------
// host dispatch
struct EltCall {
    const char* name;
    int dtype, rank, nsrc;
    nk_buf drn; const int32_t* drn_cfg;
    nk_buf src[NK_FUSE_MAX_SRC]; const int32_t* src_cfg[NK_FUSE_MAX_SRC];
    bool own[NK_FUSE_MAX_SRC];          // see LiteralArgs::own
    unsigned pin[NK_FUSE_MAX_SRC];      // see LiteralArgs::pin
    int64_t n;
};

static unsigned grid_for(Device* dev, uint64_t work_blocks) {
    uint64_t cap = (uint64_t)dev->props.multiProcessorCount * 16;
    if (cap < 256) cap = 256;
    return (unsigned)(work_blocks < cap ? (work_blocks ? work_blocks : 1) : cap);
}

template <typename T>
static int launch_typed(Device* dev, const EltCall& c, const Prog& prog) {
    Cfg cfgs[MAX_OPERANDS];
    const Cfg* cfgp[MAX_OPERANDS];
    load_cfg(cfgs[0], c.drn_cfg, c.rank);
    cfgp[0] = &cfgs[0];
    for (int j = 0; j < c.nsrc; j++) { load_cfg(cfgs[j + 1], c.src_cfg[j], c.rank); cfgp[j + 1] = &cfgs[j + 1]; }
    bool axis_on[MAX_OPERANDS][NK_MAX_RANK];
    for (int k = 0; k < NK_MAX_RANK; k++) axis_on[0][k] = true;
    for (int j = 0; j < c.nsrc; j++)
        for (int k = 0; k < NK_MAX_RANK; k++) axis_on[j + 1][k] = !((c.pin[j] >> k) & 1u);
    Ptrs ptrs{};
    for (int j = 0; j < c.nsrc; j++) ptrs.p[j] = (const void*)c.src[j];
    T* drn = (T*)c.drn;

    bool own_unravel[MAX_OPERANDS];
    own_unravel[0] = true;
    for (int j = 0; j < c.nsrc; j++) own_unravel[j + 1] = c.own[j];
    Canon cn;
    const bool canon_ok = canonicalize(cn, c.rank, cfgs[0].shape, c.nsrc + 1, cfgp, axis_on, own_unravel);
    if (!canon_ok) {
        LiteralArgs A{};
        A.rank = c.rank; A.nsrc = c.nsrc; A.n = (unsigned)c.n; A.own = 0;
        for (int j = 0; j < c.nsrc; j++) { if (c.own[j]) A.own |= 1u << j; A.pin[j] = c.pin[j]; }
        for (int o = 0; o <= c.nsrc; o++) A.cfg[o] = cfgs[o];
        set_path("literal");
        hipLaunchKernelGGL(literal_kernel<T>, dim3(grid_for(dev, (c.n + 255) / 256)), dim3(256), 0, dev->stream, A, prog, drn, ptrs);
        NK_HIP(hipGetLastError());
        return NK_OK;
    }
    if (cn.rank == 0) { cn.rank = 1; cn.shape[0] = 1; for (int o = 0; o <= c.nsrc; o++) cn.stride[o][0] = 1; }
    const int last = cn.rank - 1;
    bool rows_ok = cn.stride[0][last] == 1;
    for (int j = 0; j < c.nsrc; j++) rows_ok = rows_ok && (cn.stride[j + 1][last] == 0 || cn.stride[j + 1][last] == 1);

    if (rows_ok) {
        constexpr int VMAX = 16 / sizeof(T);
        bool vec = cn.shape[last] % VMAX == 0;
        for (int o = 0; o <= c.nsrc && vec; o++) {
            uint64_t addr = o == 0 ? c.drn : c.src[o - 1];
            if (o > 0 && cn.stride[o][last] == 0) {
                continue;   // read one element per row: no alignment needed
            }
            if (addr % 16 != 0 || cn.base[o] % VMAX != 0) vec = false;
            for (int k = 0; k < last; k++) if (cn.stride[o][k] % VMAX != 0) vec = false;
        }
        const int V = vec ? VMAX : 1;
        RowsArgs A{};
        A.rank = cn.rank; A.nsrc = c.nsrc;
        A.L = (unsigned)cn.shape[last];
        uint64_t n_rows = 1;
        for (int k = 0; k < last; k++) { n_rows *= cn.shape[k]; A.outer[k] = FastDiv((unsigned)cn.shape[k]); }
        A.n_rows = (unsigned)n_rows;
        uint64_t vec_per_row = (A.L + V - 1) / V;
        int l2 = 0;
        while ((1u << l2) < vec_per_row && l2 < 8) l2++;
        A.tpr_log2 = l2;
        const unsigned tpr = 1u << l2, rpp = 256u >> l2;
        A.chunks = (unsigned)((vec_per_row + tpr - 1) / tpr);
        A.passes = 4;
        uint64_t row_tiles = (n_rows + (uint64_t)rpp * A.passes - 1) / ((uint64_t)rpp * A.passes);
        uint64_t n_tiles = row_tiles * A.chunks;
        if (n_tiles >= ((uint64_t)1 << 31)) return set_error(NK_ERR_UNSUPPORTED, "%s: too many tiles", c.name);
        A.n_tiles = (unsigned)n_tiles;
        A.chunk_div = FastDiv(A.chunks);
        for (int o = 0; o <= c.nsrc; o++) {
            A.base[o] = cn.base[o];
            for (int k = 0; k < cn.rank; k++) A.stride[o][k] = cn.stride[o][k];
        }
        set_path(V > 1 ? "rows_vec" : "rows");
        dim3 grid(grid_for(dev, n_tiles));
        if (V > 1) hipLaunchKernelGGL((rows_kernel<T, VMAX>), grid, dim3(256), 0, dev->stream, A, prog, drn, ptrs);
        else       hipLaunchKernelGGL((rows_kernel<T, 1>),    grid, dim3(256), 0, dev->stream, A, prog, drn, ptrs);
        NK_HIP(hipGetLastError());
        return NK_OK;
    }

    // tile_transpose: the drain and some operands run along the innermost axis, the others along one
    // common outer axis
    if (cn.stride[0][last] == 1 && cn.rank >= 2) {
        int pax = -1;
        unsigned turned = 0;
        bool ok = true;
        for (int j = 0; j < c.nsrc && ok; j++) {
            int64_t sl = cn.stride[j + 1][last];
            if (sl == 0 || sl == 1) continue;
            int cand = -1;
            for (int k = 0; k < last; k++) if (cn.stride[j + 1][k] == 1) { cand = k; break; }
            if (cand < 0 || (pax >= 0 && cand != pax)) ok = false;
            else { pax = cand; turned |= 1u << j; }
        }
        if (ok && pax >= 0) {
            TileArgs A{};
            A.rank = cn.rank; A.nsrc = c.nsrc; A.pax = pax; A.turned = turned;
            A.P = (unsigned)cn.shape[pax]; A.L = (unsigned)cn.shape[last];
            A.tiles_p = (A.P + 63) / 64; A.tiles_l = (A.L + 63) / 64;
            uint64_t nb = (uint64_t)A.tiles_p * A.tiles_l;
            for (int k = 0; k < last; k++) {
                if (k == pax) continue;
                nb *= cn.shape[k];
                A.outer[k] = FastDiv((unsigned)cn.shape[k]);
            }
            if (nb < ((uint64_t)1 << 31)) {
                A.n_blocks = (unsigned)nb;
                A.div_tiles_l = FastDiv(A.tiles_l); A.div_tiles_p = FastDiv(A.tiles_p);
                for (int o = 0; o <= c.nsrc; o++) {
                    A.base[o] = cn.base[o];
                    for (int k = 0; k < cn.rank; k++) A.stride[o][k] = cn.stride[o][k];
                }
                set_path("tile_transpose");
                hipLaunchKernelGGL(tile_kernel<T>, dim3(grid_for(dev, nb)), dim3(256), 0, dev->stream, A, prog, drn, ptrs);
                NK_HIP(hipGetLastError());
                return NK_OK;
            }
        }
    }

    CanonArgs A{};
    A.rank = cn.rank; A.nsrc = c.nsrc; A.n = (unsigned)cn.n;
    for (int k = 0; k < cn.rank; k++) A.dims[k] = FastDiv((unsigned)cn.shape[k]);
    for (int o = 0; o <= c.nsrc; o++) {
        A.base[o] = cn.base[o];
        for (int k = 0; k < cn.rank; k++) A.stride[o][k] = cn.stride[o][k];
    }
    set_path("canon");
    hipLaunchKernelGGL(canon_kernel<T>, dim3(grid_for(dev, (cn.n + 255) / 256)), dim3(256), 0, dev->stream, A, prog, drn, ptrs);
    NK_HIP(hipGetLastError());
    return NK_OK;
}

static int launch_eltwise(nk_dev h, const EltCall& c, const Prog& prog) {
    NK_DEVICE(dev, h);
    NK_REQUIRE(c.dtype == NK_F32 || c.dtype == NK_F64, "%s: unknown dtype %d", c.name, c.dtype);
    if (int e = check_cfg(c.name, c.drn_cfg, c.rank)) return e;
    int64_t size = 1;
    for (int k = 0; k < c.rank; k++) size *= c.drn_cfg[k];
    NK_REQUIRE(c.n == size, "%s: n = %lld but the drain's shape holds %lld elements", c.name, (long long)c.n, (long long)size);
    NK_REQUIRE(size < ((int64_t)1 << 31), "%s: %lld elements, the limit is 2^31-1", c.name, (long long)size);
    const int eb = dtype_bytes(c.dtype);
    if (int e = check_extent(dev, c.name, c.drn, c.drn_cfg, c.rank, eb)) return e;
    for (int j = 0; j < c.nsrc; j++) {
        if (int e = check_cfg(c.name, c.src_cfg[j], c.rank)) return e;
        // sources addressed with the drain's nd-index may be smaller on pinned axes only
        if (!c.own[j])
            for (int k = 0; k < c.rank; k++)
                NK_REQUIRE(((c.pin[j] >> k) & 1u) || c.src_cfg[j][k] >= c.drn_cfg[k],
                           "%s: source %d has extent %d on axis %d, the drain has %d", c.name, j, c.src_cfg[j][k], k, c.drn_cfg[k]);
        else {
            int64_t ssz = 1;
            for (int k = 0; k < c.rank; k++) ssz *= c.src_cfg[j][k];
            NK_REQUIRE(ssz >= size, "%s: source %d holds %lld elements, the drain %lld", c.name, j, (long long)ssz, (long long)size);
        }
        if (int e = check_extent(dev, c.name, c.src[j], c.src_cfg[j], c.rank, eb)) return e;
    }
    return c.dtype == NK_F32 ? launch_typed<float>(dev, c, prog) : launch_typed<double>(dev, c, prog);
}

}  // namespace nk

using namespace nk;

extern "C" {

int nk_activation(nk_dev dev, int fun_id, int d, int dtype, int rank, nk_buf drn, const int32_t* drn_cfg,
                  nk_buf src, const int32_t* src_cfg, int64_t n) {
    NK_REQUIRE(fun_id >= 0 && fun_id < NK_FUN_COUNT, "nk_activation: unknown function id %d", fun_id);
    ProgBuilder b;
    b.emit(I_SET, 0, 0);
    b.emit(d < 0 ? I_FUN : I_DFUN, fun_id, 0);
    EltCall c{};
    c.name = "nk_activation"; c.dtype = dtype; c.rank = rank; c.nsrc = 1;
    c.drn = drn; c.drn_cfg = drn_cfg; c.src[0] = src; c.src_cfg[0] = src_cfg; c.own[0] = false; c.n = n;
    return launch_eltwise(dev, c, b.p);
}

int nk_elementwise(nk_dev dev, int op_id, int d, int dtype, int rank, nk_buf drn, const int32_t* drn_cfg,
                   nk_buf a, const int32_t* a_cfg, nk_buf b_, const int32_t* b_cfg, int64_t n) {
    NK_REQUIRE(op_id >= NK_OP_ADD && op_id <= NK_OP_POW, "nk_elementwise: unknown operator id %d", op_id);
    NK_REQUIRE(d >= -1 && d <= 1, "nk_elementwise: derivative index %d outside [-1, 1]", d);
    ProgBuilder b;
    b.emit(I_SET, 0, 0);
    if (d < 0) b.emit(I_BIN, op_id, 1);
    else b.emit(I_DBIN, op_id * 2 + d, 1);
    EltCall c{};
    c.name = "nk_elementwise"; c.dtype = dtype; c.rank = rank; c.nsrc = 2;
    c.drn = drn; c.drn_cfg = drn_cfg;
    c.src[0] = a; c.src_cfg[0] = a_cfg; c.own[0] = true;
    c.src[1] = b_; c.src_cfg[1] = b_cfg; c.own[1] = true;
    c.n = n;
    return launch_eltwise(dev, c, b.p);
}

int nk_scalarization(nk_dev dev, int op_id, int d, int dtype, int rank, nk_buf drn, const int32_t* drn_cfg,
                     nk_buf src, const int32_t* src_cfg, double value, int64_t n) {
    NK_REQUIRE(op_id >= NK_OP_ADD && op_id <= NK_OP_IDY, "nk_scalarization: unknown operator id %d", op_id);
    NK_REQUIRE(d >= -1 && d <= 1, "nk_scalarization: derivative index %d outside [-1, 1]", d);
    ProgBuilder b;
    b.p.consts[0] = value;
    b.emit(I_SET, 0, 0);
    if (d < 0) b.emit(I_BIN, op_id, SRC_CONST0);
    else b.emit(I_DBIN, op_id * 2 + d, SRC_CONST0);
    EltCall c{};
    c.name = "nk_scalarization"; c.dtype = dtype; c.rank = rank; c.nsrc = 1;
    c.drn = drn; c.drn_cfg = drn_cfg; c.src[0] = src; c.src_cfg[0] = src_cfg; c.own[0] = true; c.n = n;
    return launch_eltwise(dev, c, b.p);
}

int nk_scalar_fill(nk_dev dev, int dtype, int rank, nk_buf drn, const int32_t* drn_cfg, double value, int64_t n) {
    ProgBuilder b;
    b.p.consts[0] = value;
    b.emit(I_SET, 0, SRC_CONST0);
    EltCall c{};
    c.name = "nk_scalar_fill"; c.dtype = dtype; c.rank = rank; c.nsrc = 0;
    c.drn = drn; c.drn_cfg = drn_cfg; c.n = n;
    return launch_eltwise(dev, c, b.p);
}

int nk_fused(nk_dev dev, const int32_t* program, int n_ops, const double* consts, int n_consts, int dtype, int rank,
             nk_buf drn, const int32_t* drn_cfg, int n_src, const nk_buf* srcs, const int32_t* const* src_cfgs, int64_t n) {
    NK_REQUIRE(program != nullptr && n_ops >= 1 && n_ops <= NK_FUSE_MAX_OPS, "nk_fused: %d ops, must be in [1, %d]", n_ops, NK_FUSE_MAX_OPS);
    NK_REQUIRE(n_src >= 0 && n_src <= NK_FUSE_MAX_SRC, "nk_fused: %d sources, at most %d", n_src, NK_FUSE_MAX_SRC);
    NK_REQUIRE(n_consts >= 0 && n_consts <= NK_FUSE_MAX_CONST && (n_consts == 0 || consts), "nk_fused: %d constants, at most %d", n_consts, NK_FUSE_MAX_CONST);
    NK_REQUIRE(n_src == 0 || (srcs && src_cfgs), "nk_fused: null source arrays");
    Prog prog;
    if (int e = compile_postfix(prog, program, n_ops, consts, n_consts, n_src)) return e;
    EltCall c{};
    c.name = "nk_fused"; c.dtype = dtype; c.rank = rank; c.nsrc = n_src;
    c.drn = drn; c.drn_cfg = drn_cfg; c.n = n;
    for (int j = 0; j < n_src; j++) { c.src[j] = srcs[j]; c.src_cfg[j] = src_cfgs[j]; c.own[j] = true; }
    return launch_eltwise(dev, c, prog);
}

}  // extern "C"

// forward broadcast lives here because it is the same engine with pinned axes; the reducing
// backward is in nk_reduce.hip
namespace nk {
int broadcast_forward(nk_dev dev, int op_id, int dtype, int rank, nk_buf drn, const int32_t* drn_cfg,
                      nk_buf a, const int32_t* a_cfg, nk_buf b_, const int32_t* b_cfg, int64_t n) {
    if (int e = check_cfg("nk_broadcast", a_cfg, rank)) return e;
    if (int e = check_cfg("nk_broadcast", b_cfg, rank)) return e;
    ProgBuilder b;
    b.emit(I_SET, 0, 0);
    b.emit(I_BIN, op_id, 1);
    EltCall c{};
    c.name = "nk_broadcast"; c.dtype = dtype; c.rank = rank; c.nsrc = 2;
    c.drn = drn; c.drn_cfg = drn_cfg;
    c.src[0] = a; c.src_cfg[0] = a_cfg; c.own[0] = false;
    c.src[1] = b_; c.src_cfg[1] = b_cfg; c.own[1] = false;
    // CPUBroadcast.java:185-196: equal extents -> both follow the drain; otherwise the smaller one is pinned to 0
    for (int k = 0; k < rank; k++) {
        if (a_cfg[k] < b_cfg[k]) c.pin[0] |= 1u << k;
        if (a_cfg[k] > b_cfg[k]) c.pin[1] |= 1u << k;
    }
    c.n = n;
    return launch_eltwise(dev, c, b.p);
}
}  // namespace nk
