// Host side of the elementwise kernel family: activation, binary elementwise, scalarization, fill,
// forward broadcast and fused expressions.  All of them are "drain[i] = program(sources at i)": the
// operation is compiled to a tiny accumulator program, the view descriptors are analysed and one of four
// kernels is chosen
//   rows            every operand is contiguous (or constant) along the innermost collapsed axis:
//                   coalesced 16-byte accesses, outer axes resolved once per row
//   tile_transpose  some source is contiguous along a different axis than the drain (permuted
//                   views): 64x64 tiles are turned through LDS so both sides stay coalesced
//   canon           any other strided combination: one element per thread, mul-shift divisions
//   literal         descriptors that do not reduce to base+strides: the reference's index formula
// in the instantiation (element type x function set x source count) that fits the program.
#include "nk_eltwise.h"
#include <cstdlib>

namespace nk {

struct ProgBuilder {
    Prog p{};
    bool ok = true;
    void emit(int op, int arg, int src) {
        if (p.n >= MAX_INSTR) { ok = false; return; }
        p.op[p.n] = (unsigned char)op; p.arg[p.n] = (unsigned char)arg; p.src[p.n] = (unsigned char)src;
        p.n++;
    }
};

// smallest function set that can run the program
static int funset_of(const Prog& p) {
    bool fun = false, dfun = false, full = false;         // dfun: needs the full table (derivatives, heavy entries)
    int saved = 0;
    for (int i = 0; i < p.n; i++) {
        if (p.op[i] != I_FUN && p.op[i] != I_DFUN && p.op[i] != I_PUSH && p.src[i] == SRC_POP) saved--;
        switch (p.op[i]) {
            case I_FUN: fun = true; if (fun_is_heavy(p.arg[i])) dfun = true; break;
            case I_DFUN: dfun = true; break;
            case I_BIN: case I_RBIN: if (bin_is_heavy(p.arg[i])) dfun = true; break;
            case I_DBIN: case I_RDBIN: if (dbin_is_heavy(p.arg[i] >> 1)) dfun = true; break;
            case I_PUSH:                          // one saved intermediate: set 3; more: the long-program family
                dfun = true;
                if (++saved > 1) full = true;
                break;
            default: break;
        }
    }
    return full ? 2 : dfun ? 3 : fun ? 1 : 0;
}

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
    // One block per tile: on this part a streaming kernel is fastest when the grid is far larger than the
    // machine (262144 blocks of 256 threads write at 6.3 TB/s, 4096 grid-striding blocks at 4.6 TB/s).
    (void)dev;
    const uint64_t cap = ((uint64_t)1 << 31) - 1;
    if (work_blocks == 0) work_blocks = 1;
    return (unsigned)(work_blocks < cap ? work_blocks : cap);
}

template <typename T>
static int launch_typed(Device* dev, const EltCall& c, const Prog& prog) {
    Cfg cfgs[MAX_OPERANDS];
    const Cfg* cfgp[MAX_OPERANDS];
    load_cfg(cfgs[0], c.drn_cfg, c.rank);
    cfgp[0] = &cfgs[0];
    for (int j = 0; j < c.nsrc; j++) { load_cfg(cfgs[j + 1], c.src_cfg[j], c.rank); cfgp[j + 1] = &cfgs[j + 1]; }
    // every operand that unravels the flat index itself: a table that would leave its view becomes the row-major one
    tame_unravel(cfgs[0], c.rank, c.n);
    for (int j = 0; j < c.nsrc; j++) if (c.own[j]) tame_unravel(cfgs[j + 1], c.rank, c.n);
    bool axis_on[MAX_OPERANDS][NK_MAX_RANK];
    for (int k = 0; k < NK_MAX_RANK; k++) axis_on[0][k] = true;
    for (int j = 0; j < c.nsrc; j++)
        for (int k = 0; k < NK_MAX_RANK; k++) axis_on[j + 1][k] = !((c.pin[j] >> k) & 1u);
    bool own_unravel[MAX_OPERANDS];
    own_unravel[0] = true;
    for (int j = 0; j < c.nsrc; j++) own_unravel[j + 1] = c.own[j];

    static thread_local Plan plan;         // large (kernel argument blocks): kept off the stack
    plan = Plan{};
    plan.prog = prog;
    for (int i = 0; i < MAX_INSTR; i++)
        plan.prog.code[i] = i < prog.n ? (unsigned)prog.op[i] | ((unsigned)prog.arg[i] << 8) | ((unsigned)prog.src[i] << 16) : 0u;
    plan.nsrc = c.nsrc;
    plan.drn = (void*)c.drn;
    for (int j = 0; j < c.nsrc; j++) plan.srcs.p[j] = (const void*)c.src[j];
    int funset = funset_of(prog);
    if (c.nsrc > 3) funset = 2;            // the specialised families carry at most 3 source registers
    // ... and run the packed short form of the program
    int n_consts = 0;
    for (int i = 0; i < prog.n; i++)
        if (prog.op[i] != I_FUN && prog.op[i] != I_DFUN && prog.op[i] != I_PUSH && prog.src[i] >= SRC_CONST0 && prog.src[i] < SRC_POP)
            n_consts = n_consts > prog.src[i] - SRC_CONST0 + 1 ? n_consts : prog.src[i] - SRC_CONST0 + 1;
    // (programs of 9 to 16 instructions without derivatives also fit the derivative family, which carries set 1)
    if (n_consts > LIGHT_CONST) funset = 2;
    else if (prog.n > (funset == 3 ? LIGHT_INSTR_D : LIGHT_INSTR)) funset = (funset != 2 && prog.n <= LIGHT_INSTR_D) ? 3 : 2;
    if (funset != 2) {
        plan.light.n = prog.n;
        for (int i = 0; i < prog.n; i++) plan.light.code[i] = prog.op[i] | (prog.arg[i] << 8) | (prog.src[i] << 16);
        for (int i = 0; i < LIGHT_CONST; i++) plan.light.consts[i] = prog.consts[i];
    }
    // outputs far larger than the last-level cache are written with non-temporal stores
    // an output far larger than the caches: sources read once are loaded past them, re-used ones take the lean kernel
    const bool streaming = (uint64_t)c.n * sizeof(T) >= ((uint64_t)64 << 20);
    // the kernels with one unit per block: from 16 MiB of output on (measured: 32 MiB 8.8 -> 7.9 us; at 8 MiB no difference)
    constexpr uint64_t lean_from = (uint64_t)16 << 20;
    const bool large = (uint64_t)c.n * sizeof(T) >= lean_from;

    Canon cn;
    const bool canon_ok = canonicalize(cn, c.rank, cfgs[0].shape, c.nsrc + 1, cfgp, axis_on, own_unravel);
    if (!canon_ok) {
        LiteralArgs& A = plan.literal;
        A.rank = c.rank; A.nsrc = c.nsrc; A.n = (unsigned)c.n; A.own = 0;
        for (int j = 0; j < c.nsrc; j++) { if (c.own[j]) A.own |= 1u << j; A.pin[j] = c.pin[j]; }
        for (int o = 0; o <= c.nsrc; o++) A.cfg[o] = cfgs[o];
        plan.kind = PLAN_LITERAL;
        plan.grid = grid_for(dev, (c.n + 255) / 256);
        set_path("literal");
        return launch_family<T, 2>(dev, plan);
    }
    if (cn.rank == 0) { cn.rank = 1; cn.shape[0] = 1; for (int o = 0; o <= c.nsrc; o++) cn.stride[o][0] = 1; }
    // An innermost axis shorter than a vector (rows of three: channels-last data with a per-channel operand,
    // [.., N, 3] o [.., 1, 3]) would run one element per thread, one of up to seven elements on overlapping vectors.  Where the drain and every source are dense
    // across the innermost axis and the one above it -- or pinned on the upper one, i.e. periodic in the merged axis, or
    // constant along both -- the two axes become one long row: dense operands move in vectors, periodic ones are gathered
    // at column mod period.
    unsigned periodic = 0;
    int64_t period_of[MAX_OPERANDS] = {};
    {
        constexpr int VM = 16 / sizeof(T);
        Canon m = cn;
        unsigned per = 0;
        int64_t per_of[MAX_OPERANDS] = {};
        bool any = false;
        const int64_t first_row = m.rank >= 1 ? m.shape[m.rank - 1] : 0;
        while (m.rank >= 2) {
            const int l = m.rank - 1;
            const int64_t L = m.shape[l];
            if (L >= 2 * VM || L % VM == 0 || L < 2) break;      // longer rows run on (overlapping) vectors as they are
            bool ok = m.stride[0][l] == 1 && m.stride[0][l - 1] == L;
            unsigned per_next = per;
            for (int j = 0; j < c.nsrc && ok; j++) {
                const int64_t in = m.stride[j + 1][l], up = m.stride[j + 1][l - 1];
                if ((per >> j) & 1u) ok = up == 0;                                   // stays periodic with its period
                else if (in == 1 && up == L) {}                                      // dense across both
                else if (in == 1 && up == 0) { per_next |= 1u << j; per_of[j + 1] = L; }
                else if (in == 0 && up == 0) {}                                      // one value for the merged row
                else ok = false;
            }
            if (!ok) break;
            per = per_next;
            m.shape[l - 1] *= L;
            for (int o = 0; o <= c.nsrc; o++) m.stride[o][l - 1] = m.stride[o][l];   // 1 (dense or periodic) or 0
            m.rank--;
            any = true;
        }
        // what the rows kernels need of the merged form (they keep element offsets in 32 bits)
        // Rows of VM elements and more also run on overlapping vectors as they are; measured, the merged form wins there
        // only when everything merges into one row ([2^22,5] + [1,5]: 6.4 TB/s merged; [2^20,1,5] o [1,64,5]: 3.0 merged --
        // rows of 320 leave 48 of 128 lanes idle -- and [4096,1,5] o [1,4096,5] 4.4, against 4.9 on overlapping vectors).
        bool fits = any && per != 0 && m.rank - 1 <= ROWS_MAX_OUTER && (first_row < VM || m.rank == 1);
        for (int o = 0; o <= c.nsrc && fits; o++) {
            int64_t lo = m.base[o], hi = m.base[o];
            for (int k = 0; k < m.rank; k++) {
                const int64_t span = (m.shape[k] - 1) * m.stride[o][k];
                if (span < 0) lo += span; else hi += span;
                if (m.stride[o][k] > INT32_MAX || m.stride[o][k] < INT32_MIN) fits = false;
            }
            if (lo < INT32_MIN || hi > INT32_MAX) fits = false;
        }
        if (fits) { cn = m; periodic = per; for (int o = 0; o < MAX_OPERANDS; o++) period_of[o] = per_of[o]; }
    }
    const int last = cn.rank - 1;
    bool rows_ok = cn.stride[0][last] == 1 && cn.rank - 1 <= ROWS_MAX_OUTER;
    // sources may also take every n-th column (a gather per element; the drain is still written in whole vectors)
    for (int j = 0; j < c.nsrc; j++)
        rows_ok = rows_ok && (cn.stride[j + 1][last] == 0 || cn.stride[j + 1][last] == 1 ||
                              (cn.stride[j + 1][last] > 1 && cn.stride[j + 1][last] <= 8));
    bool done = false;

    // the rows kernel keeps element offsets in 32 bits: every reachable offset must fit
    if (rows_ok) {
        for (int o = 0; o <= c.nsrc && rows_ok; o++) {
            int64_t lo = cn.base[o], hi = cn.base[o];
            for (int k = 0; k < cn.rank; k++) {
                const int64_t span = (cn.shape[k] - 1) * cn.stride[o][k];
                if (span < 0) lo += span; else hi += span;
                if (cn.stride[o][k] > INT32_MAX || cn.stride[o][k] < INT32_MIN) rows_ok = false;
            }
            if (lo < INT32_MIN || hi > INT32_MAX) rows_ok = false;
        }
    }
    if (rows_ok) {
        constexpr int VMAX = 16 / sizeof(T);
        // 16 bytes per lane whenever a row is a whole number of vectors (no alignment requirement).  A ragged row
        // (length not a multiple of the vector) also runs on vectors: the last vector of a row is moved back so
        // that it ends with the row and overlaps its neighbour, whose elements are then computed and written twice
        // with the same values -- which is only the same thing when no source shares memory with the drain.
        bool ragged = cn.shape[last] % VMAX != 0 && cn.shape[last] >= VMAX;
        if (ragged) {
            auto span = [&](int o, int64_t& lo, int64_t& hi) {
                const int64_t ptr = o == 0 ? (int64_t)c.drn : (int64_t)c.src[o - 1];
                lo = hi = cn.base[o];
                for (int k = 0; k < cn.rank; k++) {
                    const int64_t sp = (cn.shape[k] - 1) * cn.stride[o][k];
                    if (sp < 0) lo += sp; else hi += sp;
                }
                lo = ptr + lo * (int64_t)sizeof(T); hi = ptr + (hi + 1) * (int64_t)sizeof(T);
            };
            int64_t dlo, dhi;
            span(0, dlo, dhi);
            for (int j = 0; j < c.nsrc && ragged; j++) {
                int64_t slo, shi;
                span(j + 1, slo, shi);
                if (slo < dhi && dlo < shi) ragged = false;
            }
        }
        const bool vec = cn.shape[last] % VMAX == 0 || ragged;
        RowsArgs& A = plan.rows;
        const int V = vec ? VMAX : 1;
        int passes = rows_passes(funset, funset == 2 ? NK_FUSE_MAX_SRC : (c.nsrc <= 1 ? 1 : c.nsrc));
        A.nouter = last; A.nsrc = c.nsrc;
        A.L = (unsigned)cn.shape[last];
        // sources at least as large as the drain's threshold whose every element is read once stream past the caches
        bool reused = false;                                // some source is read more than once (a broadcast)
        for (int j = 0; j < c.nsrc; j++)
            for (int k = 0; k < cn.rank; k++) if (cn.shape[k] > 1 && cn.stride[j + 1][k] == 0) reused = true;
        if (periodic) reused = true;
        bool once = streaming && !reused;
        const bool deep = last > ROWS_FAST_OUTER;           // more outer axes than the tuned variants resolve: plain variants
        if (deep) once = false;
        A.nt_loads = once ? 1 : 0;
        A.const_last = 0;
        A.strided_last = 0;
        for (int j = 0; j < c.nsrc; j++) {
            if (cn.stride[j + 1][last] == 0) A.const_last |= 1u << j;
            else if (cn.stride[j + 1][last] != 1) A.strided_last |= 1u << j;
            A.last_stride[j + 1] = (int)cn.stride[j + 1][last];
        }
        A.last_stride[0] = 1;
        A.periodic_last = periodic;
        for (int o = 0; o < MAX_OPERANDS; o++) A.period[o] = FastDiv((unsigned)(period_of[o] > 0 ? period_of[o] : 1));
        uint64_t n_rows = 1;
        // kernel axis k counts outward from the innermost outer axis
        for (int k = 0; k < last; k++) { n_rows *= cn.shape[k]; A.outer[k] = FastDiv((unsigned)cn.shape[last - 1 - k]); }
        A.n_rows = (unsigned)n_rows;
        const uint64_t vec_per_row = (A.L + V - 1) / V;
        int l2 = 0;
        while ((1u << l2) < vec_per_row && l2 < 8) l2++;
        A.tpr_log2 = l2;
        const unsigned tpr = 1u << l2;
        unsigned rpp = 256u >> l2;
        A.chunks = (unsigned)((vec_per_row + tpr - 1) / tpr);
        uint64_t row_groups = (n_rows + rpp - 1) / rpp;
        A.flat_vpr = FastDiv(1);
        if (row_groups * A.chunks >= ((uint64_t)1 << 31)) return set_error(NK_ERR_UNSUPPORTED, "%s: too many work units", c.name);
        A.row_groups = (unsigned)row_groups;
        A.chunk_div = FastDiv(A.chunks);
        for (int o = 0; o <= c.nsrc; o++) {
            A.base[o] = (int)cn.base[o];
            for (int k = 0; k < last; k++) A.stride[o][k] = (int)cn.stride[o][last - 1 - k];
        }
        A.vec = V;
        A.ragged = ragged ? 1 : 0;
        A.simple_loads = (funset != 2 && A.const_last == 0 && A.strided_last == 0 && periodic == 0 && c.nsrc >= 1 && c.nsrc <= 3) ? 1 : 0;
        plan.kind = PLAN_ROWS;
        // drain = src0 op src1 with + - * /: the dedicated kernel
        // (sources that are constant along a row are handled by that kernel's vector variant only)
        const bool loads_ok = A.simple_loads || (A.const_last != 0 && A.strided_last == 0 && periodic == 0 && vec) ||
                              ((periodic == 1 || periodic == 2) && A.const_last == 0 && A.strided_last == 0 && vec && !deep);
        if (loads_ok && c.nsrc == 2 && funset == 0 && prog.n == 2 && prog.op[0] == I_SET && prog.src[0] == 0 &&
            prog.op[1] == I_BIN && prog.src[1] == 1 && prog.arg[1] <= NK_OP_DIV) {
            plan.kind = PLAN_ROWS_BINARY;
            plan.binary_op = prog.arg[1];
            if (vec) passes = 8;
            plan.passes = passes;
        }
        plan.vec = vec;
        // Rows of fewer than 256 vectors, no power of two, leave lanes idle (33 vectors per row: 31 of 64).  From a fifth
        // of the lanes on, the threads are numbered through all rows without gaps (one division per thread instead of a
        // shift) -- from three tenths on where the launch would otherwise take the one-unit-per-block kernel, which has
        // its own addressing and is still the faster one below that when its rows end on 128-byte lines ([4096,1,96] o
        // [1,1024,96], a quarter idle: 6.35 against 5.65 TB/s; [4096,1,132] o [1,1024,132], 48 % idle: 4.17 against 5.65;
        // [4096,1,100] o [1,1024,100], 22 % idle and rows of 400 bytes: 4.9 against 5.6).
        bool dense_drain = cn.stride[0][last] == 1;
        for (int k = last - 1; k >= 0 && dense_drain; k--) dense_drain = cn.stride[0][k] == cn.stride[0][k + 1] * (int64_t)cn.shape[k + 1];
        const bool lean_candidate = plan.kind == PLAN_ROWS_BINARY && vec && large && dense_drain && !deep && A.strided_last == 0 && periodic == 0 && reused;
        const bool whole_lines = ((uint64_t)A.L * sizeof(T)) % 128 == 0;      // rows that end on a 128-byte line
        // the one-unit-per-block kernel numbers its threads through the rows as well (its drain is dense, so a block still
        // writes one contiguous aligned unit): wherever a tenth of its lanes would idle or its rows do not end on a line
        // (The sources a broadcast re-reads live in the L2 of each XCD.  Numbered by row and column chunk, the blocks an XCD
        // gets -- every eighth -- keep to the same columns, so it holds an eighth of such a source; numbered through, they
        // drift across the columns and every XCD ends up cycling through all of it.  With rows of more than a block that
        // costs more than the idle lanes once the sources exceed what one L2 keeps: [64,1,4092] o [1,1024,4092], 16 MiB
        // re-read, 5.6 -> 3.7 TB/s; 2 MiB and less, or rows of at most 256 vectors, gain: 5.4 -> 6.0 .. 6.4.)
        uint64_t reread_bytes = 0;
        for (int j = 0; j < c.nsrc; j++) {
            uint64_t elems = 1;
            bool reread = false;
            for (int k = 0; k < cn.rank; k++) { if (cn.stride[j + 1][k] != 0) elems *= (uint64_t)cn.shape[k]; else if (cn.shape[k] > 1) reread = true; }
            if (reread) reread_bytes += elems * sizeof(T);
        }
        const bool lean_flat = lean_candidate && !ragged && c.nsrc == 2 && A.const_last == 0 && n_rows * vec_per_row < ((uint64_t)1 << 31) &&
                               (!whole_lines || vec_per_row * 10 <= (uint64_t)tpr * A.chunks * 9) &&
                               (vec_per_row <= 256 || reread_bytes <= ((uint64_t)2 << 20));
        const bool flat_rows = lean_flat || (vec_per_row < 256 && n_rows * vec_per_row < ((uint64_t)1 << 31) &&
                               (lean_candidate && whole_lines ? vec_per_row * 10 <= (uint64_t)tpr * 7 : vec_per_row * 5 <= (uint64_t)tpr * 4));
        if (flat_rows) {
            A.flat_vpr = FastDiv((unsigned)vec_per_row);
            row_groups = (n_rows * vec_per_row + 255) / 256;
            A.row_groups = (unsigned)row_groups;
            A.chunks = 1; A.chunk_div = FastDiv(1);             // a unit is 256 vectors of the launch, not a piece of a row
            rpp = 0;                                            // no whole number of rows per unit: nothing below may assume one
        }
        // a source that is constant along the innermost outer axis is the same memory in every pass of a block
        // when the block's rows never straddle that axis: the binary kernel then loads it once
        plan.hoist = 0;
        A.pass_rows = 0;
        if (plan.kind == PLAN_ROWS_BINARY && last >= 1 && row_groups >= (uint64_t)passes) {
            int constant = 0;
            for (int j = 0; j < 2; j++) if (cn.stride[j + 1][last - 1] == 0) constant |= 1 << j;
            if (constant && !flat_rows) A.pass_rows = 1;
            // measured at steady state: loading the constant source once gains 2..14 % when a row fills the block
            // (256 threads) and loses 4..14 % when a block covers several rows per pass
            if (constant && vec && passes == 8 && !A.nt_loads && rpp == 1 && A.const_last == 0 && !deep &&
                cn.shape[last - 1] % ((int64_t)passes * rpp) == 0)
                plan.hoist = constant;
        }
        // one block per `passes` units, no grid-stride loop
        plan.grid = A.pass_rows ? (unsigned)(((row_groups + passes - 1) / passes) * A.chunks)
                                : (unsigned)((row_groups * A.chunks + passes - 1) / passes);
        // large outputs of the binary kernel: one unit per block, non-temporal stores
        // (only for a drain without gaps: the gain comes from the write front that moves through memory in order; a
        // drain that is a slice of a wider tensor measured 5 % slower this way)
        bool drain_dense = cn.stride[0][last] == 1;
        for (int k = last - 1; k >= 0 && drain_dense; k--) drain_dense = cn.stride[0][k] == cn.stride[0][k + 1] * (int64_t)cn.shape[k + 1];
        if (plan.kind == PLAN_ROWS_BINARY && vec && large && drain_dense && !deep && A.strided_last == 0 && periodic == 0 && reused && (!flat_rows || lean_flat)) {
            plan.lean = true;
            plan.hoist = 0;
            plan.grid = (unsigned)(row_groups * A.chunks);
        }
        // ... and of a program that is one constant
        if (plan.kind == PLAN_ROWS && c.nsrc == 0 && prog.n == 1 && prog.op[0] == I_SET && prog.src[0] == SRC_CONST0 && funset == 0 &&
            vec && large && drain_dense && !deep && !flat_rows) {
            plan.lean_fill = true;
            plan.fill_value = prog.consts[0];
            plan.grid = (unsigned)(row_groups * A.chunks);
        }
        // ... and of a program that is one function (or one derivative) of its one source: the kernel with that function
        // compiled in.  Its blocks take two units each, whatever the interpreter family of the program would take.
        if (plan.kind == PLAN_ROWS && c.nsrc == 1 && prog.n == 2 && prog.op[0] == I_SET && prog.src[0] == 0 &&
            (prog.op[1] == I_FUN || prog.op[1] == I_DFUN) && prog.arg[1] < NK_FUN_COUNT && vec && A.simple_loads && !deep) {
            plan.single = true;
            plan.single_deriv = prog.op[1] == I_DFUN;
            plan.single_fun = prog.arg[1];
            plan.grid = (unsigned)((row_groups * A.chunks + SINGLE_PASSES - 1) / SINGLE_PASSES);
        }
        // ... and of one heavy operator (or its derivative) of source 0 and either source 1 or a constant
        if (plan.kind == PLAN_ROWS && (c.nsrc == 1 || c.nsrc == 2) && prog.n == 2 && prog.op[0] == I_SET && prog.src[0] == 0 &&
            (prog.op[1] == I_BIN || prog.op[1] == I_DBIN) && vec && A.simple_loads && !deep &&
            (prog.src[1] == SRC_CONST0 || (prog.src[1] == 1 && c.nsrc == 2)) && (prog.src[1] == 1) == (c.nsrc == 2)) {
            const int op = prog.op[1] == I_BIN ? prog.arg[1] : prog.arg[1] >> 1;
            const int kind = prog.op[1] == I_BIN ? 0 : 1 + (prog.arg[1] & 1);
            if (kind == 0 ? bin_is_heavy(op) : dbin_is_heavy(op)) {
                plan.single = true;
                plan.pair_kind = kind; plan.pair_op = op;
                plan.pair_const = prog.src[1] == SRC_CONST0;
                plan.pair_value = prog.consts[0];
                plan.grid = (unsigned)((row_groups * A.chunks + SINGLE_PASSES - 1) / SINGLE_PASSES);
            }
        }
        set_path(plan.single ? (plan.pair_kind >= 0 ? "rows_vec_pair" : "rows_vec_single") : plan.lean_fill ? "rows_vec_fill_lean" : plan.lean ? "rows_vec_binary_lean"
                           : plan.kind == PLAN_ROWS_BINARY ? (periodic ? "rows_vec_binary_periodic" : vec ? "rows_vec_binary" : "rows_binary")
                           : periodic ? (vec ? "rows_vec_periodic" : "rows_periodic") : vec ? "rows_vec" : "rows");
        done = true;
    }

    // tile_transpose: the drain and some operands run along the innermost axis, the others along one
    // common outer axis
    if (!done && funset != 2 && cn.stride[0][last] == 1 && cn.rank >= 2) {
        int pax = -1;
        unsigned turned = 0;
        bool ok = true;
        for (int j = 0; j < c.nsrc && ok; j++) {
            const int64_t sl = cn.stride[j + 1][last];
            if (sl == 0 || sl == 1) continue;
            int cand = -1;
            for (int k = 0; k < last; k++) if (cn.stride[j + 1][k] == 1) { cand = k; break; }
            if (cand < 0 || (pax >= 0 && cand != pax)) ok = false;
            else { pax = cand; turned |= 1u << j; }
        }
        if (ok && pax >= 0) {
            TileArgs& A = plan.tile;
            A.rank = cn.rank; A.nsrc = c.nsrc; A.pax = pax; A.turned = turned;
            bool once = streaming;
            for (int j = 0; j < c.nsrc && once; j++)
                for (int k = 0; k < cn.rank; k++) if (cn.shape[k] > 1 && cn.stride[j + 1][k] == 0) once = false;
            A.nt_loads = once ? 1 : 0;
            A.careful = 0;
            for (int j = 0; j < c.nsrc; j++)
                if (!((turned >> j) & 1u) && cn.stride[j + 1][last] == 0) A.careful = 1;
            A.P = (unsigned)cn.shape[pax]; A.L = (unsigned)cn.shape[last];
            A.tiles_p = (A.P + TILE_P - 1) / TILE_P; A.tiles_l = (A.L + TILE_L - 1) / TILE_L;
            uint64_t nb = (uint64_t)A.tiles_p * A.tiles_l;
            for (int k = 0; k < last; k++) {
                if (k == pax) continue;
                nb *= cn.shape[k];
                A.outer[k] = FastDiv((unsigned)cn.shape[k]);
            }
            if (nb < ((uint64_t)1 << 31)) {
                A.n_blocks = (unsigned)nb;
                // groups of 4 (pax) x 8 (innermost) tiles: 1 KiB runs on both sides (f32); measured optimum of the sweep
                int gl = 3, gp = 2;
                while (gl > 0 && A.tiles_l % (1u << gl)) gl--;
                while (gp > 0 && A.tiles_p % (1u << gp)) gp--;
                A.group_log2 = gl; A.group_p_log2 = gp;
                A.div_tiles_l = FastDiv(A.tiles_l >> gl); A.div_tiles_p = FastDiv(A.tiles_p >> gp);
                for (int o = 0; o <= c.nsrc; o++) {
                    A.base[o] = cn.base[o];
                    for (int k = 0; k < cn.rank; k++) A.stride[o][k] = cn.stride[o][k];
                }
                plan.kind = PLAN_TILE;
                plan.grid = (unsigned)nb;                    // one block per tile
                // The hardware deals consecutive block ids round-robin to the 8 XCDs, each with its own L2.  XCD x takes the
                // x-th eighth of the tile order, so the tiles one L2 serves at a time are neighbours in both directions:
                // its reads (along pax) and its writes (along the innermost axis) add up to long runs
                // (with fewer than 8 tiles in a plane the order is ruled by the outer axes and an eighth per XCD is an eighth of
                // the output per XCD, which a write stream does not like: measured 5.5 -> 4.7 TB/s on a fully reversed rank-4 view)
                A.xcd_regions = nb % 8 == 0 && (uint64_t)A.tiles_p * A.tiles_l >= 8;
                set_path("tile_transpose");
                done = true;
            }
        }
    }

    if (!done) {
        CanonArgs& A = plan.canon;
        A.rank = cn.rank; A.nsrc = c.nsrc; A.n = (unsigned)cn.n;
        for (int k = 0; k < cn.rank; k++) A.dims[k] = FastDiv((unsigned)cn.shape[k]);
        for (int o = 0; o <= c.nsrc; o++) {
            A.base[o] = cn.base[o];
            for (int k = 0; k < cn.rank; k++) A.stride[o][k] = cn.stride[o][k];
        }
        plan.kind = PLAN_CANON;
        plan.grid = grid_for(dev, (cn.n + 255) / 256);
        set_path("canon");
    }
    if (plan.single) return launch_single<T>(dev, plan);
    switch (funset) {
        case 0: return launch_family<T, 0>(dev, plan);
        case 1: return launch_family<T, 1>(dev, plan);
        case 3: return launch_family<T, 3>(dev, plan);
        default: return launch_family<T, 2>(dev, plan);
    }
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
    // x ** 2 is the correctly rounded product (exact in double for a float x, what Math.pow returns) and x ** 1 is x by
    // Math.pow's specification: both leave the heavy power kernels for the streaming ones
    if (d < 0 && op_id == NK_OP_POW && value == 2.0) b.emit(I_BIN, NK_OP_MUL, 0);
    else if (d < 0 && op_id == NK_OP_POW && value == 1.0) { /* a copy */ }
    else if (d < 0) b.emit(I_BIN, op_id, SRC_CONST0);
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
