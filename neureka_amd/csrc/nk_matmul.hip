// Dense matrix multiplication C[M,N] += A[M,K] @ B[K,N].
//
//   mfma_big f32, M % 256 == 0, N % 256 == 0, K % 32 == 0, K >= 1024 and enough 256x256 tiles to fill the compute
//            units in whole rounds: one block per compute unit, one wavefront per SIMD with 4x4 accumulators.
//   mfma_big_edge  the same kernel for large shapes that are not whole tiles: clamped edges, zeroed k tail.
//   mfma     f32, M % 128 == 0, N % 128 == 0, K % 32 == 0: 128x128 block tiles, four wavefronts in a
//            2x2 arrangement, each owning a 64x64 sub-tile as 2x2 v_mfma_f32_32x32x2_f32
//            accumulators; A and B k-slices of depth 32 are staged through double-buffered LDS with
//            register prefetch of the next slice.  Block ids are regrouped so that the blocks that
//            are co-resident on one XCD (block id mod 8) form a compact patch of the tile grid
//            and share A row panels and B column panels in that XCD's L2.
//   mfma_edge  the same kernel for f32 shapes that are not whole tiles, from 2^24 multiply-adds on: clamped
//            edges, zeroed k tail, element-wise stores along the edges.
//   mfma_f64 / mfma_f64_edge  f64 from 2^24 multiply-adds on: v_mfma_f64_16x16x4_f64, same tiling.
//   ..._split  the same kernels for products with fewer tiles than compute units: the k range cut into parts,
//            partial tiles in the device workspace, added in order by a second launch.
//   ..._bands  a few more tiles than whole rounds of the machine: two row bands, the lower one in parts of its k range.
//   mfma_mixed / mfma_edge_mixed  f32, a few more tiles than whole rounds of one per compute unit: one launch whose
//            upper tile rows take the whole k range and whose lower rows come as parts of it.
//   mfma_stream  f32 whole tiles with at most eight k-slices and many tiles: blocks that stay and walk the tiles.
//   mfma_tiles_of_64, mfma_f64_tiles_of_64 (…_edge, …_split, …_mixed)  64x64 block tiles, chosen by an estimate of the
//            time: products with few large tiles, with a last round of large tiles that would idle most units, narrow
//            results over long k ranges (every tile in parts), k ranges of a few slices.
//   few_rows / few_cols / some_cols / short_inner  products that stream one large operand once (a batch of up to 32
//            rows or 16 columns, K <= 16): no matrix-core tiles, the large operand read once at the memory rate.
//   simple   everything else (small products): one thread per element of C, the k loop in the
//            reference's order with the product rounded before the add, which makes it bit-identical
//            to GEMM.partial_F32_MxN_RM + AXPY (J/backend/main/operations/linear/internal/blas/GEMM.java:282-304,
//            AXPY.java:47-59).
//
// Column-major operands are handled as the transposed row-major problem C^T = B^T A^T.
#include "nk_internal.h"
#include <mutex>
#include <type_traits>

namespace nk {

template <typename T>
__global__ __launch_bounds__(256) void matmul_simple_kernel(int M, int K, int N, int overwrite, const T* __restrict__ A,
                                                            const T* __restrict__ B, T* __restrict__ C) {
    const int n = blockIdx.x * 64 + (threadIdx.x & 63);
    const int m = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (m >= M || n >= N) return;
    T acc = overwrite ? T(0) : C[(int64_t)m * N + n];
    const T* a = A + (int64_t)m * K;
    for (int k = 0; k < K; k++) {
        T prod = a[k] * B[(int64_t)k * N + n];   // rounded product, then add: no contraction
        acc = acc + prod;
    }
    C[(int64_t)m * N + n] = acc;
}

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int BM = 128, BN = 128, BK = 32;
constexpr int A_PITCH = BK + 4;     // floats; keeps 16-byte alignment of every row
constexpr int B_PITCH = BN + 4;

struct MfmaArgs {
    int M, K, N;
    int tiles_m, tiles_n;
    int group_rows;      // tile rows per group of the block-id regrouping
    int splits;          // SPLIT kernels: parts the k range is cut into (grid = tiles * splits) ...
    int split_slices;    // ... and k-slices per part
    int overwrite;       // C = A @ B instead of C += A @ B: the old values of C are not read
    int rows_a;          // MIXED kernels: tile rows whose tiles take the whole k range (the rest: parts, as in SPLIT)
};

__device__ __forceinline__ void tile_of_block(const MfmaArgs& g, int bid, int& tm, int& tn) {
    // hardware deals consecutive block ids round-robin to the 8 XCDs: give XCD x the x-th contiguous
    // eighth of a grouped ordering (groups of `group_rows` tile rows, walked column by column)
    const int nblk = g.tiles_m * g.tiles_n;
    int logical = bid;
    if (nblk % 8 == 0) logical = (bid % 8) * (nblk / 8) + bid / 8;
    const int per_group = g.group_rows * g.tiles_n;
    const int grp = logical / per_group;
    const int first_row = grp * g.group_rows;
    int rows = g.tiles_m - first_row;
    if (rows > g.group_rows) rows = g.group_rows;
    const int in_grp = logical - grp * per_group;
    tm = first_row + in_grp % rows;
    tn = in_grp / rows;
}

// ---- what the f32 tile kernels share ---------------------------------------------------------------------------------
// A block of 256 threads stages one k-slice (depth BK = 32) of a TM x TN tile -- A as TM rows of BK floats, B as BK rows
// of TN floats, N_STAGED 16-byte pieces of each per thread -- through registers into LDS; a wavefront owns RI x RJ tiles
// of 32 x 32 and reads the operands of a chunk of depth 8 as RI 16-byte pieces of A and RJ x 4 floats of B.  Lane half h
// owns k = 8c + 4h ... + 3 of chunk c; the four multiply-adds of a chunk pair (k, k + 4): any pairing works as long as A
// and B use the same one.  Row pitches in LDS keep every row 16-byte aligned and the operand reads free of bank conflicts.
// The kernels differ in their pipelines (how far ahead a slice is requested, where the barrier sits, the pinned order
// of issue), not in any of this.  (matmul_mfma64_kernel, whose order of issue is left to the compiler, keeps its own copy
// of the staging: through this helper the compiler's schedule changed and 1024^3 ran 3 % slower.)
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
template <int TM, int TN, int RI, int RJ>
struct TileF32 {
    static_assert(TM == TN, "one thread stages as many pieces of A as of B");
    static constexpr int A_P = BK + 4, B_P = TN + 4;
    static constexpr int N_STAGED = TM * BK / 1024;
    static constexpr int B_STEP = 1024 / TN;                 // rows of B between two pieces of one thread
    static constexpr int A_FLOATS = TM * A_P, B_FLOATS = BK * B_P;
    struct Staged { f32x4 a[N_STAGED], b[N_STAGED]; };
    struct Frag {
        f32x4 a[RI];           // rows wm + 32 i + l32, k = 8c + 4h .. + 3
        float b[RJ][4];        // [j][t]: column wn + 32 j + l32, k = 8c + 4h + t
    };
    int a_row, a_col, b_row, b_col;      // a thread's pieces: rows a_row + 32 i of A, rows b_row + B_STEP i of B
    __device__ __forceinline__ explicit TileF32(int tid) : a_row(tid >> 3), a_col((tid & 7) * 4), b_row(tid / (TN / 4)), b_col((tid % (TN / 4)) * 4) {}
    // Whole tiles: Ag = the tile's first row of A, Bg = its first column of B.  A lane's byte offsets inside a slice are
    // the same for the whole k loop (offsets(), kept in registers); the slice moves the base of two buffer descriptors,
    // which is scalar arithmetic -- with a 64-bit address per load the vector unit spent two additions on each of them
    // between the multiply-adds (4096^3: 941 -> 914 us).  (TM x K and 32 x N floats stay below the 2 GiB the descriptors span.)
    struct Offsets { unsigned a[N_STAGED], b[N_STAGED]; };
    __device__ __forceinline__ Offsets offsets(int K, int N) const {
        Offsets o;
#pragma unroll
        for (int i = 0; i < N_STAGED; i++) {
            o.a[i] = (unsigned)(((a_row + 32 * i) * K + a_col) * 4);
            o.b[i] = (unsigned)(((b_row + B_STEP * i) * N + b_col) * 4);
        }
        return o;
    }
    __device__ __forceinline__ void request(Staged& s, const Offsets& o, const float* Ag, const float* Bg, int N, int k0) const {
        const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void*)(Ag + k0), 0, 0x80000000u, 0x00020000);
        const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void*)(Bg + (int64_t)k0 * N), 0, 0x80000000u, 0x00020000);
#pragma unroll
        for (int i = 0; i < N_STAGED; i++) {
            s.a[i] = __builtin_bit_cast(f32x4, (u32x4)__builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ra, o.a[i], 0, 0)));
            s.b[i] = __builtin_bit_cast(f32x4, (u32x4)__builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rb, o.b[i], 0, 0)));
        }
    }
    // any shape: through buffer descriptors that end where the matrices end (nothing past their end is touched, the range
    // check returns 0 there); rows past the edge are clamped, columns past the edge left as they come: all of these only
    // feed results that are not stored, once zero_tail has cleared the k tail
    // (offsets of a lane's pieces from the first element of the matrices, rows past the edge clamped: fixed for the k loop)
    __device__ __forceinline__ Offsets edge_offsets(int M, int K, int N, int row0, int col0) const {
        Offsets o;
#pragma unroll
        for (int i = 0; i < N_STAGED; i++) {
            int row = row0 + a_row + 32 * i; if (row > M - 1) row = M - 1;
            o.a[i] = (unsigned)(row * K + a_col) * 4u;
            o.b[i] = (unsigned)((b_row + B_STEP * i) * N + col0 + b_col) * 4u;
        }
        return o;
    }
    // the slice in the base of the descriptors, which end where the matrices end: k rows of B past the end read as 0
    __device__ __forceinline__ void request_edge(Staged& s, const Offsets& o, const float* A, const float* B, int M, int K, int N, int k0) const {
        const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void*)(A + k0), 0, (unsigned)(((int64_t)M * K - k0) * 4), 0x00020000);
        const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void*)(B + (int64_t)k0 * N), 0, (unsigned)((int64_t)(K - k0) * N * 4), 0x00020000);
#pragma unroll
        for (int i = 0; i < N_STAGED; i++) {
            s.a[i] = __builtin_bit_cast(f32x4, (u32x4)__builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ra, o.a[i], 0, 0)));
            s.b[i] = __builtin_bit_cast(f32x4, (u32x4)__builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rb, o.b[i], 0, 0)));
        }
    }
    __device__ __forceinline__ void zero_tail(Staged& s, int K, int k0) const {
#pragma unroll
        for (int i = 0; i < N_STAGED; i++) {
#pragma unroll
            for (int e = 0; e < 4; e++) if (k0 + a_col + e >= K) s.a[i][e] = 0.0f;
            if (k0 + b_row + B_STEP * i >= K) s.b[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
    }
    __device__ __forceinline__ void store(const Staged& s, float* as, float* bs) const {
#pragma unroll
        for (int i = 0; i < N_STAGED; i++) {
            *(f32x4*)(&as[(a_row + 32 * i) * A_P + a_col]) = s.a[i];
            *(f32x4*)(&bs[(b_row + B_STEP * i) * B_P + b_col]) = s.b[i];
        }
    }
    static __device__ __forceinline__ void read(Frag& f, const float* as, const float* bs, int wm, int wn, int l32, int h, int c) {
#pragma unroll
        for (int i = 0; i < RI; i++) f.a[i] = *(const f32x4*)(&as[(wm + 32 * i + l32) * A_P + 8 * c + 4 * h]);
#pragma unroll
        for (int t = 0; t < 4; t++)
#pragma unroll
            for (int j = 0; j < RJ; j++) f.b[j][t] = bs[(8 * c + 4 * h + t) * B_P + wn + 32 * j + l32];
    }
    static __device__ __forceinline__ void clear(f32x16 (&acc)[RI][RJ]) {
#pragma unroll
        for (int i = 0; i < RI; i++)
#pragma unroll
            for (int j = 0; j < RJ; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;
    }
    static __device__ __forceinline__ void mma(f32x16 (&acc)[RI][RJ], const Frag& f) {
#pragma unroll
        for (int t = 0; t < 4; t++)
#pragma unroll
            for (int i = 0; i < RI; i++)
#pragma unroll
                for (int j = 0; j < RJ; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(f.a[i][t], f.b[j][t], acc[i][j], 0, 0, 0);
    }
};
using Tile128 = TileF32<BM, BN, 2, 2>;       // matmul_mfma_kernel, matmul_mfma_stream_kernel: 64 x 64 per wavefront
static_assert(Tile128::A_P == A_PITCH && Tile128::B_P == B_PITCH, "one LDS layout");

constexpr int C_PITCH = BN + 4;
constexpr int LDS_FLOATS_AB = 2 * BM * A_PITCH + 2 * BK * B_PITCH;
constexpr int LDS_FLOATS_C = BM * C_PITCH;
constexpr int LDS_FLOATS = LDS_FLOATS_AB > LDS_FLOATS_C ? LDS_FLOATS_AB : LDS_FLOATS_C;

// EDGE: M, N, K need not be multiples of the tile.  Loads go through buffer descriptors over the whole
// matrices (nothing past their end is touched, the range check returns 0 there), rows and columns past the
// edge are clamped or left as they come (they only feed results that are not stored), and the k tail is zeroed
// in both operands so that it adds exactly nothing; the epilogue stores element-wise along the edges.
// SPLIT: few tiles (small or thin products): the k range is cut into g.splits parts, block (tile, part) stores its
// partial tile to P[part] instead of adding it to C, and matmul_add_parts_kernel adds the parts in order.
// MIXED: one launch for a product with more tiles than compute units but fewer than the blocks that fit the machine (two
// per unit): the blocks of the first g.rows_a tile rows come first and take a whole tile each, about one per unit; the
// tiles of the remaining rows follow as parts of their k range, as in SPLIT, written to P (a matrix of those rows
// only) and added by matmul_add_parts.  The short blocks fill the second place on every unit as they come and go, so
// the units finish together instead of some with one tile and some with two.
template <bool EDGE, bool SPLIT = false, bool MIXED = false>
__global__ __launch_bounds__(256) void matmul_mfma_kernel(MfmaArgs g, const float* __restrict__ A,
                                                          const float* __restrict__ B, float* __restrict__ C, float* __restrict__ P = nullptr) {
    static_assert(!MIXED || !SPLIT, "the mixed launch splits part of an unsplit product itself");
    __shared__ __attribute__((aligned(16))) float lds[LDS_FLOATS];
    float* const As0 = lds;                                   // [2][BM * A_PITCH]
    float* const Bs0 = lds + 2 * BM * A_PITCH;                // [2][BK * B_PITCH]

    int tm, tn;
    const int n_tiles = g.tiles_m * g.tiles_n;
    int part = SPLIT ? (int)blockIdx.x / n_tiles : 0;
    bool parted = SPLIT;                                      // this block computes a part of its tile's k range, into P
    if constexpr (MIXED) {
        const int tiles_a = g.rows_a * g.tiles_n;
        MfmaArgs band = g;
        if ((int)blockIdx.x < tiles_a) {
            band.tiles_m = g.rows_a;
            band.group_rows = g.group_rows < band.tiles_m ? g.group_rows : band.tiles_m;
            tile_of_block(band, (int)blockIdx.x, tm, tn);
        } else {
            band.tiles_m = g.tiles_m - g.rows_a;
            band.group_rows = g.group_rows < band.tiles_m ? g.group_rows : band.tiles_m;
            const int tiles_b = band.tiles_m * g.tiles_n, b = (int)blockIdx.x - tiles_a;
            part = b / tiles_b;
            tile_of_block(band, b - part * tiles_b, tm, tn);
            tm += g.rows_a;
            parted = true;
        }
    } else {
        tile_of_block(g, SPLIT ? (int)blockIdx.x - part * n_tiles : (int)blockIdx.x, tm, tn);
    }
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;     // wave's sub-tile origin inside the block tile
    const int l32 = lane & 31, h = lane >> 5;

    const float* Ag = A + (int64_t)tm * BM * g.K;
    const float* Bg = B + (int64_t)tn * BN;

    const Tile128 tile(tid);
    Tile128::Staged staged;
    const Tile128::Offsets offs = EDGE ? tile.edge_offsets(g.M, g.K, g.N, tm * BM, tn * BN) : tile.offsets(g.K, g.N);
    auto load_global = [&](int k0) {
        if (!EDGE) tile.request(staged, offs, Ag, Bg, g.N, k0);
        else tile.request_edge(staged, offs, A, B, g.M, g.K, g.N, k0);
    };
    // k0: the slice the staging registers hold.  The k tail is zeroed here, a slice after the request, and only in the one
    // slice that has a tail (a block-uniform branch): zeroed at the request, every slice would wait for its loads there
    // (2000^3: 205 us so, against 146 for 2048^3).
    auto store_lds = [&](int buf, int k0) {
        if (EDGE && k0 + BK > g.K) tile.zero_tail(staged, g.K, k0);
        tile.store(staged, As0 + buf * Tile128::A_FLOATS, Bs0 + buf * Tile128::B_FLOATS);
    };
    using Frag = Tile128::Frag;
    auto read_frag = [&](Frag& f, int buf, int c) { Tile128::read(f, As0 + buf * Tile128::A_FLOATS, Bs0 + buf * Tile128::B_FLOATS, wm, wn, l32, h, c); };
    f32x16 acc[2][2];
    Tile128::clear(acc);
    auto mma = [&](const Frag& f) { Tile128::mma(acc, f); };

    // Software pipeline over the k-slices.  While the matrix cores work on chunk c of the current slice the
    // operands of chunk c + 1 are read from LDS; the next slice (fetched from global memory at the top of
    // the slice) is written to the other LDS buffer in the middle of the slice; the single barrier sits
    // before the last chunk's multiply-adds, which then cover the read of the next slice's first chunk.
    // A buffer is rewritten only after a barrier that every wavefront reaches with all its reads of that
    // buffer complete.
    static_assert(BK == 32, "the pipeline below is written for four depth-8 chunks per slice");
    const int all_slices = (g.K + BK - 1) / BK;
    const int slice0 = parted ? part * g.split_slices : 0;                          // first k-slice of this block
    int nk = all_slices;                                                             // ... and how many it takes
    if (parted) { nk = all_slices - slice0; if (nk > g.split_slices) nk = g.split_slices; }
    const int kbase = slice0 * BK;
    Frag f0, f1;
    load_global(kbase);
    store_lds(0, kbase);
    load_global(kbase + (nk > 1 ? BK : 0));                // slice 1 waits in the staging registers
    __syncthreads();
    read_frag(f0, 0, 0);
    // The order of issue inside a chunk is pinned with scheduling groups.  Left alone, the compiler sinks the LDS
    // reads of chunk c + 1 behind the sixteen multiply-adds of chunk c (fewer live registers), and the matrix cores
    // then sit out an LDS latency at the start of every chunk.  Pinned: the six reads follow the first three
    // multiply-adds, global requests and LDS writes are dealt out one per multiply-add after them, so every memory
    // instruction issues in the shadow of a multiply-add and has the rest of the chunk to complete.
#define NK_MFMA(n) __builtin_amdgcn_sched_group_barrier(0x008, n, 0)
#define NK_DS_READ(n) __builtin_amdgcn_sched_group_barrier(0x100, n, 0)
#define NK_DS_WRITE(n) __builtin_amdgcn_sched_group_barrier(0x200, n, 0)
#define NK_VMEM_READ(n) __builtin_amdgcn_sched_group_barrier(0x020, n, 0)
#define NK_FENCE __builtin_amdgcn_sched_barrier(0)
#define NK_READS_FIRST NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2)
#define NK_CHUNK_PLAIN NK_READS_FIRST; NK_MFMA(13); NK_FENCE
#define NK_CHUNK_WITH(GROUP) NK_READS_FIRST; NK_MFMA(1); GROUP(1); NK_MFMA(1); GROUP(1); NK_MFMA(1); GROUP(1); NK_MFMA(1); GROUP(1); \
                             NK_MFMA(1); GROUP(1); NK_MFMA(1); GROUP(1); NK_MFMA(1); GROUP(1); NK_MFMA(1); GROUP(1); NK_MFMA(5); NK_FENCE
#define NK_CHUNK_WRITE_AND_REQUEST NK_READS_FIRST; NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); \
                                   NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); \
                                   NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); \
                                   NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); NK_MFMA(5); NK_FENCE
    NK_FENCE;
    // Slice kt + 1 is written to LDS in the third chunk of slice kt from the staging registers, which are then free
    // for the request of slice kt + 2: a request has a whole slice of multiply-adds to arrive.  (Past the last slice
    // the request repeats the last one; nothing reads it.)
    for (int kt = 0; kt + 1 < nk; kt++) {                  // branch-free body; the last slice is peeled off below
        const int cur = kt & 1;
        read_frag(f1, cur, 1);
        mma(f0);
        NK_CHUNK_PLAIN;
        read_frag(f0, cur, 2);
        mma(f1);
        NK_CHUNK_PLAIN;
        read_frag(f1, cur, 3);                             // (before the writes in program order: LDS accesses keep it)
        store_lds(cur ^ 1, kbase + (kt + 1) * BK);
        load_global(kbase + (kt + 2 < nk ? kt + 2 : nk - 1) * BK);
        mma(f0);
        NK_CHUNK_WRITE_AND_REQUEST;
        __syncthreads();
        NK_FENCE;
        read_frag(f0, cur ^ 1, 0);
        mma(f1);
        NK_CHUNK_PLAIN;
    }
    {
        const int cur = (nk - 1) & 1;
        read_frag(f1, cur, 1);
        mma(f0);
        NK_CHUNK_PLAIN;
        read_frag(f0, cur, 2);
        mma(f1);
        NK_CHUNK_PLAIN;
        read_frag(f1, cur, 3);
        mma(f0);
        NK_CHUNK_PLAIN;
        mma(f1);
    }

    // epilogue: the block's 128x128 result goes through LDS so that C is read and written in 16-byte pieces
    // along its rows; accumulator v of a 32x32 tile sits at row 8*(v/4) + 4*h + v%4, column l32
    __syncthreads();
    float* cs = lds;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = wm + 32 * i + 8 * (v >> 2) + 4 * h + (v & 3);
                cs[row * C_PITCH + wn + 32 * j + l32] = acc[i][j][v];
            }
    __syncthreads();
    float* Cg = C + (int64_t)tm * BM * g.N + tn * BN;
    if (parted) Cg = P + ((int64_t)part * (g.M - (MIXED ? g.rows_a * BM : 0)) + (int64_t)(tm - (MIXED ? g.rows_a : 0)) * BM) * g.N + tn * BN;
    const int c_col = (tid & 31) * 4, c_row = tid >> 5;
    if (EDGE) {
        const int rows = g.M - tm * BM, cols = g.N - tn * BN;          // what is left of C from this tile's origin
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int r = c_row + 8 * i;
            if (r < rows) {
                const float* add = &cs[r * C_PITCH + c_col];
                float* dst = Cg + (int64_t)r * g.N + c_col;
#pragma unroll
                for (int e = 0; e < 4; e++) if (c_col + e < cols) dst[e] = (parted || g.overwrite) ? add[e] : dst[e] + add[e];
            }
        }
        return;
    }
    if (parted || g.overwrite) {                           // the same for every thread of a block
#pragma unroll
        for (int i = 0; i < 16; i++)
            *(f32x4*)(Cg + (int64_t)(c_row + 8 * i) * g.N + c_col) = *(const f32x4*)(&cs[(c_row + 8 * i) * C_PITCH + c_col]);
        return;
    }
    f32x4 old[16];
#pragma unroll
    for (int i = 0; i < 16; i++) old[i] = *(const f32x4*)(Cg + (int64_t)(c_row + 8 * i) * g.N + c_col);
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const f32x4 add = *(const f32x4*)(&cs[(c_row + 8 * i) * C_PITCH + c_col]);
        *(f32x4*)(Cg + (int64_t)(c_row + 8 * i) * g.N + c_col) = old[i] + add;
    }
}

// Products with fewer 128 x 128 tiles than compute units (1024^3 has 64) but enough 64 x 64 tiles to give every unit
// one: 64 x 64 block tiles over the whole k range, four wavefronts in a 2 x 2 arrangement with one 32 x 32 accumulator
// each.  One launch and no partial tiles, where cutting the k range of the large tiles into parts pays for a second launch
// and for writing and re-reading the parts.  A lane feeds a multiply-add two registers per 64 cycles, so a single
// wavefront per SIMD keeps its matrix core busy through the loads and the one barrier of a k-slice.  Whole tiles only
// (M % 64 == 0, N % 64 == 0, K % 32 == 0, 16-byte aligned operands); the result leaves straight from the accumulators
// (32 lanes cover 128 contiguous bytes of a row of C).
namespace t64 {
constexpr int TM = 64, TN = 64;
constexpr int A_P = BK + 4, B_P = TN + 4;                    // floats; rows stay 16-byte aligned
constexpr int STAGE = TM * A_P + BK * B_P;                   // one k-slice of A and of B
constexpr int LDS_FLOATS = 3 * STAGE;
}
// EDGE: any M, N, K and any (element-aligned) operands, as in the larger kernels: offsets from the first element of the
// matrices with the rows past the edge clamped, descriptors that end where the matrices end (k rows of B past the end
// read as 0), the k tail of A zeroed at the LDS write of the one slice that has it, stores guarded element by element.
// MIXED (as in matmul_mfma_kernel): the blocks of the first g.rows_a tile rows come first and take a whole tile each; the
// tiles of the remaining rows follow as g.splits parts of their k range, written to P (a matrix of those rows only), which
// matmul_add_parts adds into C.
template <bool MIXED>
__device__ __forceinline__ void small_tile_of_block(const MfmaArgs& g, int& tm, int& tn, int& part, bool& parted) {
    if constexpr (MIXED) {
        const int tiles_a = g.rows_a * g.tiles_n;
        MfmaArgs band = g;
        if ((int)blockIdx.x < tiles_a) {
            band.tiles_m = g.rows_a;
            band.group_rows = g.group_rows < band.tiles_m ? g.group_rows : band.tiles_m;
            tile_of_block(band, (int)blockIdx.x, tm, tn);
        } else {
            band.tiles_m = g.tiles_m - g.rows_a;
            band.group_rows = g.group_rows < band.tiles_m ? g.group_rows : band.tiles_m;
            const int tiles_b = band.tiles_m * g.tiles_n, b = (int)blockIdx.x - tiles_a;
            part = b / tiles_b;
            tile_of_block(band, b - part * tiles_b, tm, tn);
            tm += g.rows_a;
            parted = true;
        }
    } else {
        tile_of_block(g, (int)blockIdx.x, tm, tn);
    }
}
template <bool OVERWRITE, bool EDGE = false, bool MIXED = false>
__global__ __launch_bounds__(256) void matmul_mfma64_kernel(MfmaArgs g, const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C,
                                                            float* __restrict__ P = nullptr) {
    using namespace t64;
    __shared__ __attribute__((aligned(16))) float lds[t64::LDS_FLOATS];
    int tm, tn, part = 0;
    bool parted = false;                                      // this block computes a part of its tile's k range, into P
    small_tile_of_block<MIXED>(g, tm, tn, part, parted);
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
    const int l32 = lane & 31, h = lane >> 5;
    const float* Ag = A + (int64_t)tm * TM * g.K;
    const float* Bg = B + (int64_t)tn * TN;
    const int a_row = tid >> 3, a_col = (tid & 7) * 4;      // rows a_row + 32 * i
    const int b_row = tid >> 4, b_col = (tid & 15) * 4;     // rows b_row + 16 * i
    f32x4 ra[2], rb[2];
    // (fixed byte offsets per lane, the slice in the base of the descriptors: see TileF32::request)
    unsigned off_a[2], off_b[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        if (EDGE) {
            int row = tm * TM + a_row + 32 * i; if (row > g.M - 1) row = g.M - 1;
            off_a[i] = (unsigned)(row * g.K + a_col) * 4u;
            off_b[i] = (unsigned)((b_row + 16 * i) * g.N + tn * TN + b_col) * 4u;
        } else {
            off_a[i] = (unsigned)(((a_row + 32 * i) * g.K + a_col) * 4);
            off_b[i] = (unsigned)(((b_row + 16 * i) * g.N + b_col) * 4);
        }
    }
    auto load_global = [&](int k0) {
        const __amdgpu_buffer_rsrc_t da = EDGE ? __builtin_amdgcn_make_buffer_rsrc((void*)(A + k0), 0, (unsigned)(((int64_t)g.M * g.K - k0) * 4), 0x00020000)
                                               : __builtin_amdgcn_make_buffer_rsrc((void*)(Ag + k0), 0, 0x80000000u, 0x00020000);
        const __amdgpu_buffer_rsrc_t db = EDGE ? __builtin_amdgcn_make_buffer_rsrc((void*)(B + (int64_t)k0 * g.N), 0, (unsigned)((int64_t)(g.K - k0) * g.N * 4), 0x00020000)
                                               : __builtin_amdgcn_make_buffer_rsrc((void*)(Bg + (int64_t)k0 * g.N), 0, 0x80000000u, 0x00020000);
#pragma unroll
        for (int i = 0; i < 2; i++) {
            ra[i] = __builtin_bit_cast(f32x4, (u32x4)__builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(da, off_a[i], 0, 0)));
            rb[i] = __builtin_bit_cast(f32x4, (u32x4)__builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(db, off_b[i], 0, 0)));
        }
    };
    // k0: the slice the staging registers hold (EDGE: its k tail is zeroed here, in the one slice that has it)
    auto store_lds = [&](int stage, int k0) {
        if (EDGE && k0 + BK > g.K) {
#pragma unroll
            for (int i = 0; i < 2; i++) {
#pragma unroll
                for (int e = 0; e < 4; e++) if (k0 + a_col + e >= g.K) ra[i][e] = 0.0f;
                if (k0 + b_row + 16 * i >= g.K) rb[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
        float* as = lds + stage * STAGE;
        float* bs = as + TM * A_P;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            *(f32x4*)(&as[(a_row + 32 * i) * A_P + a_col]) = ra[i];
            *(f32x4*)(&bs[(b_row + 16 * i) * B_P + b_col]) = rb[i];
        }
    };
    // operands of one depth-8 chunk: lane half h owns k = 8c + 4h .. + 3; the four multiply-adds pair (k, k + 4) in both operands
    struct Chunk { f32x4 a; float b[4]; };
    auto read_chunk = [&](Chunk& f, int stage, int c) {
        const float* as = lds + stage * STAGE;
        const float* bs = as + TM * A_P;
        f.a = *(const f32x4*)(&as[(wm + l32) * A_P + 8 * c + 4 * h]);
#pragma unroll
        for (int t = 0; t < 4; t++) f.b[t] = bs[(8 * c + 4 * h + t) * B_P + wn + l32];
    };
    // two accumulators that take the multiply-adds of a pair of chunks in turn: no multiply-add waits for the one before it
    f32x16 acc0, acc1;
#pragma unroll
    for (int v = 0; v < 16; v++) { acc0[v] = 0.0f; acc1[v] = 0.0f; }
    auto mma = [&](const Chunk& even, const Chunk& odd) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(even.a[t], even.b[t], acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(odd.a[t], odd.b[t], acc1, 0, 0, 0);
        }
    };
    // Three stages of LDS.  During slice kt the block writes slice kt + 2 and reads slice kt; the barrier at the end of a
    // slice publishes the writes one slice before anybody reads them, so the first chunks of slice kt + 1 are read before
    // that barrier, behind the last multiply-adds of slice kt: no wavefront starts a slice by waiting for LDS, which the
    // single wavefront of a SIMD could hide behind nothing.
    const int all_slices = (g.K + BK - 1) / BK;
    const int slice0 = parted ? part * g.split_slices : 0;                           // first k-slice of this block ...
    int nk = all_slices;                                                             // ... and how many it takes
    if (parted) { nk = all_slices - slice0; if (nk > g.split_slices) nk = g.split_slices; }
    auto clamped = [&](int slice) { return (slice0 + (slice < nk ? slice : nk - 1)) * BK; };     // past the end: the last slice again, read by nobody
    load_global(clamped(0));
    store_lds(0, clamped(0));
    load_global(clamped(1));
    store_lds(1, clamped(1));
    load_global(clamped(2));                                  // slice 2 waits in the staging registers
    __syncthreads();
    Chunk f0, f1, f2, f3;
    read_chunk(f0, 0, 0);
    read_chunk(f1, 0, 1);
    int cur = 0;                                              // stage of slice kt
    // The body is branch-free, and the write of slice kt + 2 with the request of slice kt + 3 sits in the middle of the
    // slice: at its top the wait for the request would hold up the multiply-adds behind it.  (Measured and not kept:
    // requests four slices ahead in four register sets behind a barrier that waits for LDS only -- 74 against 78 TFLOP/s
    // at 1024^3; the compiler's placement of the LDS reads between the multiply-adds decides, not the distance.)
    for (int kt = 0; kt < nk; kt++) {
        const int next = cur == 2 ? 0 : cur + 1, write = next == 2 ? 0 : next + 1;      // stages of slices kt + 1, kt + 2
        read_chunk(f2, cur, 2);
        read_chunk(f3, cur, 3);
        mma(f0, f1);
        // The order of issue is pinned (left to the compiler, the reads of chunks 2 and 3 sat right before their first use
        // and the reads of the next slice right before the barrier: 0.71 of the matrix rate in the k loop, 0.84 pinned).
        // The six LDS reads of chunks 2 and 3 behind the first three multiply-adds of chunks 0 and 1 ...
        NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(5); NK_FENCE;
        store_lds(write, clamped(kt + 2));
        load_global(clamped(kt + 3));
        read_chunk(f0, next, 0);
        read_chunk(f1, next, 1);
        mma(f2, f3);
        // ... one LDS write and one request behind each of the next four, the reads of the next slice behind three more
        NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1);
        NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_FENCE;
        __syncthreads();
        cur = next;
    }
    f32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = acc0[v] + acc1[v];
    // accumulator v sits at row 8 * (v / 4) + 4 * h + v % 4, column l32 of the wavefront's 32 x 32 tile
    float* Cg = C + (int64_t)(tm * TM + wm) * g.N + tn * TN + wn + l32;
    if (parted) Cg = P + ((int64_t)part * (g.M - g.rows_a * TM) + (int64_t)((tm - g.rows_a) * TM + wm)) * g.N + tn * TN + wn + l32;
    const int rows = g.M - (tm * TM + wm), cols = g.N - (tn * TN + wn + l32);      // EDGE: what is left of C from the lane's first element
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const int r = 8 * (v >> 2) + 4 * h + (v & 3);
        if (!EDGE || (r < rows && cols > 0)) {
            float* p = Cg + (int64_t)r * g.N;
            *p = (OVERWRITE || parted) ? acc[v] : *p + acc[v];
        }
    }
}

// Whole tiles, no split, more tiles than resident blocks: blocks that stay.  A block walks the tiles blockIdx.x,
// + gridDim.x, ... and the software pipeline over the k-slices runs on across them: the first slice of the next
// tile is fetched and written to the free LDS buffer during the last slice of the current one, so only the
// block's very first slice is waited for.  The result leaves straight from the accumulators (32 lanes cover 128
// contiguous bytes of a row of C), which needs neither LDS nor a barrier and so does not disturb the pipeline.
template <bool OVERWRITE>
__global__ __launch_bounds__(256, 2) void matmul_mfma_stream_kernel(MfmaArgs g, const float* __restrict__ A,
                                                                 const float* __restrict__ B, float* __restrict__ C) {
    __shared__ __attribute__((aligned(16))) float lds[LDS_FLOATS_AB];
    float* const As0 = lds;
    float* const Bs0 = lds + 2 * BM * A_PITCH;
    const int n_tiles = g.tiles_m * g.tiles_n;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
    const int l32 = lane & 31, h = lane >> 5;
    const Tile128 stage(tid);
    Tile128::Staged staged;
    const Tile128::Offsets offs = stage.offsets(g.K, g.N);
    auto load_global = [&](int tm, int tn, int k0) { stage.request(staged, offs, A + (int64_t)tm * BM * g.K, B + (int64_t)tn * BN, g.N, k0); };
    auto store_lds = [&](int buf) { stage.store(staged, As0 + buf * Tile128::A_FLOATS, Bs0 + buf * Tile128::B_FLOATS); };
    using Frag = Tile128::Frag;
    auto read_frag = [&](Frag& f, int buf, int c) { Tile128::read(f, As0 + buf * Tile128::A_FLOATS, Bs0 + buf * Tile128::B_FLOATS, wm, wn, l32, h, c); };
    f32x16 acc[2][2];
    auto clear = [&]() { Tile128::clear(acc); };
    auto mma = [&](const Frag& f) { Tile128::mma(acc, f); };
    static_assert(BK == 32, "the pipeline below is written for four depth-8 chunks per slice");
    const int nk = g.K / BK;

    int tile = blockIdx.x;
    if (tile >= n_tiles) return;
    int tm, tn;
    tile_of_block(g, tile, tm, tn);
    Frag f0, f1;
    clear();
    load_global(tm, tn, 0);
    store_lds(0);
    __syncthreads();
    read_frag(f0, 0, 0);
    int phase = 0;                                         // LDS buffer that holds slice 0 of the current tile
    for (;;) {
        for (int kt = 0; kt + 1 < nk; kt++) {              // as in matmul_mfma_kernel
            const int cur = (kt + phase) & 1;
            load_global(tm, tn, (kt + 1) * BK);
            read_frag(f1, cur, 1);
            mma(f0);
            read_frag(f0, cur, 2);
            mma(f1);
            store_lds(cur ^ 1);
            read_frag(f1, cur, 3);
            mma(f0);
            __syncthreads();
            read_frag(f0, cur ^ 1, 0);
            mma(f1);
        }
        // last slice of this tile; the first slice of the next tile takes the place of "slice kt + 1"
        const int cur = (nk - 1 + phase) & 1;
        const int next = tile + (int)gridDim.x;
        const bool more = next < n_tiles;                  // the same for the whole block
        int nm = tm, nn = tn;
        if (more) { tile_of_block(g, next, nm, nn); load_global(nm, nn, 0); }
        // C (+)= the tile: accumulator v of a 32x32 tile sits at row 8*(v/4) + 4*h + v%4, column l32, so a store
        // instruction writes 128 contiguous bytes of two rows.  (With the operands of the multiply-adds swapped a lane
        // would own four neighbouring columns of one row and C could move 16 bytes per lane, 32 bytes per row and
        // instruction: measured slower, 76.3 against 72.8 us for 65536 x 256 x 256.)  Addresses are a wave-uniform part
        // (tile, sub-tile, accumulator: scalar registers) plus one 32-bit offset per lane.  Accumulating, the old values
        // of the upper two sub-tiles are requested before the last multiply-adds, those of the lower two while the
        // upper two are stored.
        float* const Cg = C + (int64_t)tm * BM * g.N + tn * BN;
        const unsigned lane_off = (unsigned)((wm + 4 * h) * g.N + wn + l32);
        float old[2][16];
        auto fetch_old = [&](int i) {
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) old[j][v] = OVERWRITE ? 0.0f : (Cg + (int64_t)(32 * i + 8 * (v >> 2) + (v & 3)) * g.N + 32 * j)[lane_off];
        };
        auto store_new = [&](int i) {
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) (Cg + (int64_t)(32 * i + 8 * (v >> 2) + (v & 3)) * g.N + 32 * j)[lane_off] = OVERWRITE ? acc[i][j][v] : old[j][v] + acc[i][j][v];
        };
        fetch_old(0);
        read_frag(f1, cur, 1);
        mma(f0);
        read_frag(f0, cur, 2);
        mma(f1);
        if (more) store_lds(cur ^ 1);
        read_frag(f1, cur, 3);
        mma(f0);
        __syncthreads();
        if (more) read_frag(f0, cur ^ 1, 0);
        mma(f1);
        store_new(0);
        fetch_old(1);
        store_new(1);
        if (!more) break;
        clear();
        tile = next; tm = nm; tn = nn;
        phase = cur ^ 1;
    }
}

// Large products whose 256x256 tiles fill the machine: one block per compute unit, ONE wavefront per SIMD that owns
// 128x128 of the block's 256x256 tile as 4x4 accumulators (256 accumulation registers) -- the layout the part's 512
// registers per lane are made for.  Against the 128x128 kernel (two blocks of 64x64 wavefronts per compute unit) a
// multiply-add needs half the LDS traffic, a slice of depth 32 is 256 multiply-adds per wavefront between barriers
// instead of 64, and no second block competes for the matrix core in the same phase.  Same fragments, same order of
// the k steps inside a chunk: the sums are those of matmul_mfma_kernel bit for bit.  LDS: two buffers of
// A 256 x 36 and B 32 x 260 floats, 137 KiB (dynamic).
namespace big {
constexpr int TM = 256, TN = 256;
using Tile = TileF32<TM, TN, 4, 4>;                      // 128 x 128 per wavefront
constexpr int LDS_FLOATS = 2 * Tile::A_FLOATS + 2 * Tile::B_FLOATS;
using BigFrag = Tile::Frag;
}

// EDGE: M, N, K need not be multiples of the tile -- as in matmul_mfma_kernel<true>: loads through buffer descriptors
// over the whole matrices, rows past the edge clamped, columns past it left as they come (both only feed results that
// are not stored), the k tail zeroed in both operands, element-wise guarded stores.
template <bool OVERWRITE, bool EDGE = false>
__global__ __launch_bounds__(256, 1) void matmul_mfma_big_kernel(MfmaArgs g, const float* __restrict__ A,
                                                                const float* __restrict__ B, float* __restrict__ C) {
    using namespace big;
    extern __shared__ __attribute__((aligned(16))) float big_lds[];
    float* const As0 = big_lds;                            // [2][Tile::A_FLOATS]
    float* const Bs0 = big_lds + 2 * Tile::A_FLOATS;       // [2][Tile::B_FLOATS]
    int tm, tn;
    tile_of_block(g, (int)blockIdx.x, tm, tn);
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = (wave >> 1) * 128, wn = (wave & 1) * 128;
    const int l32 = lane & 31, h = lane >> 5;
    const float* Ag = A + (int64_t)tm * TM * g.K;
    const float* Bg = B + (int64_t)tn * TN;
    const Tile tile(tid);
    Tile::Staged staged;
    const typename Tile::Offsets offs = EDGE ? tile.edge_offsets(g.M, g.K, g.N, tm * TM, tn * TN) : tile.offsets(g.K, g.N);
    auto load_global = [&](int k0) {
        if (!EDGE) tile.request(staged, offs, Ag, Bg, g.N, k0);
        else tile.request_edge(staged, offs, A, B, g.M, g.K, g.N, k0);
    };
    // k0: the slice the staging registers hold.  The k tail is zeroed here, a slice after the request, and only in the
    // one slice that has a tail (a block-uniform branch): zeroing at the request would make every slice wait for its loads.
    auto store_lds = [&](int buf, int k0) {
        if (EDGE && k0 + BK > g.K) tile.zero_tail(staged, g.K, k0);
        tile.store(staged, As0 + buf * Tile::A_FLOATS, Bs0 + buf * Tile::B_FLOATS);
    };
    auto read_frag = [&](BigFrag& f, int buf, int c) { Tile::read(f, As0 + buf * Tile::A_FLOATS, Bs0 + buf * Tile::B_FLOATS, wm, wn, l32, h, c); };
    f32x16 acc[4][4];
    Tile::clear(acc);
    auto mma = [&](const BigFrag& f) { Tile::mma(acc, f); };
    // The pipeline of matmul_mfma_kernel with chunks of 64 multiply-adds: the 20 LDS reads of chunk c + 1 follow the
    // first ten multiply-adds of chunk c in pairs; in the third chunk each of the next sixteen multiply-adds is
    // followed by one LDS write of the staged slice kt + 1 and one global request for slice kt + 2.
#define NK_BIG_READS NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); \
                     NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2)
#define NK_BIG_PLAIN NK_BIG_READS; NK_MFMA(54); NK_FENCE
#define NK_BIG_WR4 NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1)
#define NK_BIG_WRITE_AND_REQUEST NK_BIG_READS; NK_BIG_WR4; NK_BIG_WR4; NK_BIG_WR4; NK_BIG_WR4; NK_MFMA(38); NK_FENCE
    const int nk = (g.K + BK - 1) / BK;
    BigFrag f0, f1;
    load_global(0);
    store_lds(0, 0);
    load_global(nk > 1 ? BK : 0);                          // slice 1 waits in the staging registers
    __syncthreads();
    read_frag(f0, 0, 0);
    NK_FENCE;
    for (int kt = 0; kt + 1 < nk; kt++) {
        const int cur = kt & 1;
        read_frag(f1, cur, 1);
        mma(f0);
        NK_BIG_PLAIN;
        read_frag(f0, cur, 2);
        mma(f1);
        NK_BIG_PLAIN;
        read_frag(f1, cur, 3);
        store_lds(cur ^ 1, (kt + 1) * BK);
        load_global((kt + 2 < nk ? kt + 2 : nk - 1) * BK);
        mma(f0);
        NK_BIG_WRITE_AND_REQUEST;
        __syncthreads();
        NK_FENCE;
        read_frag(f0, cur ^ 1, 0);
        mma(f1);
        NK_BIG_PLAIN;
    }
    {
        const int cur = (nk - 1) & 1;
        read_frag(f1, cur, 1);
        mma(f0);
        NK_BIG_PLAIN;
        read_frag(f0, cur, 2);
        mma(f1);
        NK_BIG_PLAIN;
        read_frag(f1, cur, 3);
        mma(f0);
        NK_BIG_PLAIN;
        mma(f1);
    }
    // The result leaves straight from the accumulators: accumulator v of a 32x32 tile sits at row 8*(v/4) + 4*h + v%4,
    // column l32, so a store instruction writes 128 contiguous bytes of two rows; the address is a wave-uniform part
    // plus one 32-bit offset per lane.  Accumulating, the old values of one row of four sub-tiles are requested together.
    float* const Cg = C + (int64_t)tm * TM * g.N + tn * TN;
    const unsigned lane_off = (unsigned)((wm + 4 * h) * g.N + wn + l32);
    if (EDGE && ((tm + 1) * TM > g.M || (tn + 1) * TN > g.N)) {       // a tile on the edge (the same for the whole block)
        const int rows = g.M - tm * TM - (wm + 4 * h), cols = g.N - tn * TN - (wn + l32);   // what is left of C from the lane's first element
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float old[4][16];
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int r = 32 * i + 8 * (v >> 2) + (v & 3);
                    old[j][v] = (OVERWRITE || r >= rows || 32 * j >= cols) ? 0.0f : (Cg + (int64_t)r * g.N + 32 * j)[lane_off];
                }
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int r = 32 * i + 8 * (v >> 2) + (v & 3);
                    if (r < rows && 32 * j < cols) (Cg + (int64_t)r * g.N + 32 * j)[lane_off] = OVERWRITE ? acc[i][j][v] : old[j][v] + acc[i][j][v];
                }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float old[4][16];
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) old[j][v] = OVERWRITE ? 0.0f : (Cg + (int64_t)(32 * i + 8 * (v >> 2) + (v & 3)) * g.N + 32 * j)[lane_off];
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) (Cg + (int64_t)(32 * i + 8 * (v >> 2) + (v & 3)) * g.N + 32 * j)[lane_off] = OVERWRITE ? acc[i][j][v] : old[j][v] + acc[i][j][v];
    }
}

// C[i] += (or, overwriting, =) part_0[i] + part_1[i] + ... in that order (the parts of a SPLIT product)
template <typename T>
__global__ __launch_bounds__(256) void matmul_add_parts_kernel(int64_t n, int parts, int overwrite, const T* __restrict__ P, T* __restrict__ C) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    // eight parts are requested before the first is added (one after the other, a thread waits out a trip to memory per part)
    T s = T(0);
    int k = 0;
    for (; k + 8 <= parts; k += 8) {
        T v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = P[(int64_t)(k + u) * n + i];
#pragma unroll
        for (int u = 0; u < 8; u++) s = (k + u == 0) ? v[u] : s + v[u];
    }
    for (; k < parts; k++) s = (k == 0) ? P[i] : s + P[(int64_t)k * n + i];
    C[i] = overwrite ? s : C[i] + s;
}
// ... 16 bytes per thread where the element count divides and C is aligned (the parts lie in the workspace): a quarter of
// the instructions for the same bytes
template <typename T>
__global__ __launch_bounds__(256) void matmul_add_parts_vec_kernel(int64_t nv, int parts, int overwrite, const T* __restrict__ P, T* __restrict__ C) {
    constexpr int VEC = 16 / (int)sizeof(T);
    typedef T Vec __attribute__((ext_vector_type(VEC)));
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nv) return;
    const Vec* Pv = (const Vec*)P;
    Vec s = Vec(T(0));
    int k = 0;
    for (; k + 8 <= parts; k += 8) {
        Vec v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = Pv[(int64_t)(k + u) * nv + i];
#pragma unroll
        for (int u = 0; u < 8; u++) s = (k + u == 0) ? v[u] : s + v[u];
    }
    for (; k < parts; k++) s = (k == 0) ? Pv[i] : s + Pv[(int64_t)k * nv + i];
    Vec* dst = (Vec*)C + i;
    *dst = overwrite ? s : *dst + s;
}
template <typename T>
static void launch_add_parts(Device* dev, int64_t n, int parts, int overwrite, const T* P, T* C) {
    constexpr int VEC = 16 / (int)sizeof(T);
    if (n % VEC == 0 && (uint64_t)C % 16 == 0 && (uint64_t)P % 16 == 0) {
        const int64_t nv = n / VEC;
        hipLaunchKernelGGL(matmul_add_parts_vec_kernel<T>, dim3((unsigned)((nv + 255) / 256)), dim3(256), 0, dev->stream, nv, parts, overwrite, P, C);
    } else {
        hipLaunchKernelGGL(matmul_add_parts_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, dev->stream, n, parts, overwrite, P, C);
    }
}

// ---- a few rows times a large matrix ----------------------------------------------------------------------------
// C[M,N] = A[M,K] @ B[K,N] with M <= 4 (a vector or a handful of rows times a weight matrix; 5 to 32 rows take
// matmul_few_rows_mfma_kernel further down, which shares this kernel's launch shape): the product reads B once
// and is bound by that stream; a 128 x 128 tile would spend its matrix cores on rows that do not exist.  A block owns
// 64 * (16 bytes / element) columns and one part of the k range (at most few_kp(MR) rows), whose piece of A it stages
// in LDS; each of its four wavefronts takes a quarter of the part -- a row of B is one contiguous kilobyte for a
// wavefront, eight rows are requested before the first is used and the next eight while these are -- with MR
// accumulators per column in registers (the elements of A come as 16-byte LDS reads of one address for the whole
// wavefront), the wavefronts meet in LDS in a fixed order, and the block's partial rows go to P[part];
// matmul_add_parts_kernel adds the parts in order.
constexpr int few_kp(int mr) { return mr <= 4 ? 1024 : mr <= 16 ? 256 : 128; }     // k rows a block stages of A: at most 16 KiB of LDS
__device__ __forceinline__ float fma_of(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double fma_of(double a, double b, double c) { return __builtin_fma(a, b, c); }
template <typename T, int MR>
__global__ __launch_bounds__(256) void matmul_few_rows_kernel(int M, int K, int N, int k_per_part, int col_blocks, const T* __restrict__ A,
                                                              const T* __restrict__ B, T* __restrict__ P) {
    constexpr int VEC = 16 / (int)sizeof(T);
    constexpr int UNROLL = 8;
    constexpr int KP = few_kp(MR);
    typedef T Vec __attribute__((ext_vector_type(VEC)));
    typedef T Quad __attribute__((ext_vector_type(4)));
    constexpr int MEET_SLOTS = MR <= 16 ? 3 : 1;                        // 32 rows: the wavefronts meet one after the other
    constexpr int A_ELEMS = MR * KP, MEET_ELEMS = MEET_SLOTS * MR * 64 * VEC;
    __shared__ __attribute__((aligned(16))) T lds[A_ELEMS > MEET_ELEMS ? A_ELEMS : MEET_ELEMS];
    T (*As)[KP] = (T (*)[KP])lds;                                       // [MR][KP], zero past the part's end
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int part = (int)(blockIdx.x / (unsigned)col_blocks), col_block = (int)(blockIdx.x % (unsigned)col_blocks);
    const int64_t col0 = ((int64_t)col_block * 64 + lane) * VEC;             // N % VEC == 0 (the host checks)
    const bool live = col0 < N;
    const int k_begin = part * k_per_part;
    const int k_count = k_begin + k_per_part < K ? k_per_part : K - k_begin;  // 1 ... KP
    const T* Bc = B + (live ? col0 : 0);
    // the wavefront's quarter of the part, a multiple of UNROLL rows long
    const int quarter = ((k_per_part + 4 * UNROLL - 1) / (4 * UNROLL)) * UNROLL;
    const int kk_end = (wave + 1) * quarter < k_count ? (wave + 1) * quarter : k_count;
    auto request = [&](Vec (&b)[UNROLL], int kk) {
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const int row = kk + u < kk_end ? kk + u : kk_end - 1;      // (what a repeated last row brings is dropped below)
            b[u] = *(const Vec*)(Bc + (int64_t)(k_begin + row) * N);
        }
    };
    Vec b[UNROLL];
    int kk = wave * quarter;
    if (kk < kk_end) request(b, kk);                                    // in flight while the piece of A is staged
    {
        // thread t stages columns t, t + 256, ... of the piece: independent loads along the rows of A
        const int t = threadIdx.x;
        constexpr int CPT = (KP + 255) / 256;                           // columns per thread
        T av[CPT][MR];
#pragma unroll
        for (int c = 0; c < CPT; c++)
#pragma unroll
            for (int m = 0; m < MR; m++) av[c][m] = A[(int64_t)(m < M ? m : M - 1) * K + k_begin + (t + 256 * c < k_count ? t + 256 * c : 0)];
#pragma unroll
        for (int c = 0; c < CPT; c++)
#pragma unroll
            for (int m = 0; m < MR; m++)
                if (t + 256 * c < KP) As[m][t + 256 * c] = (m < M && t + 256 * c < k_count) ? av[c][m] : T(0);
    }
    __syncthreads();
    T acc[MR][VEC];
#pragma unroll
    for (int m = 0; m < MR; m++)
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[m][e] = T(0);
    for (; kk < kk_end; kk += UNROLL) {
        Vec bn[UNROLL];
        if (kk + UNROLL < kk_end) request(bn, kk + UNROLL);             // the next rows, while these are used
#pragma unroll
        for (int u = 0; u < UNROLL; u++)
            if (kk + u >= kk_end) b[u] = Vec(T(0));                     // (only at the part's ragged end, where A is zero too)
#pragma unroll
        for (int q = 0; q < UNROLL; q += 4)
#pragma unroll
            for (int m = 0; m < MR; m++) {
                const Quad a = *(const Quad*)&As[m][kk + q];
#pragma unroll
                for (int u = 0; u < 4; u++)
#pragma unroll
                    for (int e = 0; e < VEC; e++) acc[m][e] = fma_of(a[u], b[q + u][e], acc[m][e]);
            }
#pragma unroll
        for (int u = 0; u < UNROLL; u++) b[u] = bn[u];
    }
    __syncthreads();                                                    // the staged piece of A makes room for the meeting
    T (*meet)[MR][64 * VEC] = (T (*)[MR][64 * VEC])lds;
    if constexpr (MEET_SLOTS == 3) {
        if (wave > 0) {
#pragma unroll
            for (int m = 0; m < MR; m++) *(Vec*)&meet[wave - 1][m][lane * VEC] = *(const Vec*)acc[m];
        }
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int m = 0; m < MR; m++)
#pragma unroll
                for (int w = 0; w < 3; w++) *(Vec*)acc[m] = *(const Vec*)acc[m] + *(const Vec*)&meet[w][m][lane * VEC];
        }
    } else {
        for (int w = 1; w < 4; w++) {
            if (wave == w) {
#pragma unroll
                for (int m = 0; m < MR; m++) *(Vec*)&meet[0][m][lane * VEC] = *(const Vec*)acc[m];
            }
            __syncthreads();
            if (wave == 0) {
#pragma unroll
                for (int m = 0; m < MR; m++) *(Vec*)acc[m] = *(const Vec*)acc[m] + *(const Vec*)&meet[0][m][lane * VEC];
            }
            __syncthreads();
        }
    }
    if (wave == 0 && live) {
        T* Pp = P + (int64_t)part * M * N + col0;
#pragma unroll
        for (int m = 0; m < MR; m++)
            if (m < M) *(Vec*)(Pp + (int64_t)m * N) = *(const Vec*)acc[m];
    }
}

// ---- a large matrix times a few columns -----------------------------------------------------------------------
// C[M,NC] = A[M,K] @ B[K,NC] with NC = 1, 2 or 4 (a weight matrix times a vector): one stream over A.  A wavefront owns R rows
// of A; its lanes walk along k with 16-byte loads (a row is read in contiguous kilobytes), every lane keeps R x NC
// sums over its own k's -- the few elements of B it needs for them are 16-byte loads of a matrix that stays in the
// caches -- and the 64 lanes' sums meet through wavefront shuffles at the end.  One launch, no partial results.
template <typename T, int NC, int R, bool OVERWRITE>
__global__ __launch_bounds__(256) void matmul_few_cols_kernel(int M, int K, const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C) {
    constexpr int VEC = 16 / (int)sizeof(T);
    constexpr int U = R == 1 ? 4 : 1;                                   // contiguous kilobytes of a row per trip (one row per wavefront: few
                                                                        // wavefronts, each must keep more in flight)
    typedef T Vec __attribute__((ext_vector_type(VEC)));
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t row0 = ((int64_t)blockIdx.x * 4 + wave) * R;
    if (row0 >= M) return;                                              // (whole wavefronts; the kernel has no barrier)
    const T* rows[R];
#pragma unroll
    for (int r = 0; r < R; r++) rows[r] = A + (row0 + r < M ? row0 + r : M - 1) * (int64_t)K;
    T acc[R][NC];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int n = 0; n < NC; n++) acc[r][n] = T(0);
    constexpr int STEP = U * 64 * VEC;                                  // k's per trip of the wavefront
    // K % VEC == 0 (the host checks): a lane's VEC k's are inside the matrix or all outside
    auto request = [&](Vec (&a)[U][R], Vec (&b)[U][NC], int k0) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = k0 + (u * 64 + lane) * VEC;
            const int kc = k < K ? k : 0;
#pragma unroll
            for (int r = 0; r < R; r++) a[u][r] = *(const Vec*)(rows[r] + kc);
            // elements [k .. k + VEC) x [0 .. NC) of B are VEC * NC contiguous values: NC vectors
#pragma unroll
            for (int j = 0; j < NC; j++) b[u][j] = *(const Vec*)(B + (int64_t)kc * NC + j * VEC);
            if (k >= K) {
#pragma unroll
                for (int r = 0; r < R; r++) a[u][r] = Vec(T(0));
#pragma unroll
                for (int j = 0; j < NC; j++) b[u][j] = Vec(T(0));
            }
        }
    };
    Vec a[U][R], b[U][NC];
    request(a, b, 0);
    for (int k0 = 0; k0 < K; k0 += STEP) {
        Vec an[U][R], bn[U][NC];
        if (k0 + STEP < K) request(an, bn, k0 + STEP);
#pragma unroll
        for (int u = 0; u < U; u++) {
            // b as a flat run f[v * NC + n]
            T f[VEC * NC];
#pragma unroll
            for (int j = 0; j < NC; j++)
#pragma unroll
                for (int e = 0; e < VEC; e++) f[j * VEC + e] = b[u][j][e];
#pragma unroll
            for (int v = 0; v < VEC; v++)
#pragma unroll
                for (int n = 0; n < NC; n++) {
                    const T bv = f[v * NC + n];
#pragma unroll
                    for (int r = 0; r < R; r++) acc[r][n] = fma_of(a[u][r][v], bv, acc[r][n]);
                }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
#pragma unroll
            for (int r = 0; r < R; r++) a[u][r] = an[u][r];
#pragma unroll
            for (int j = 0; j < NC; j++) b[u][j] = bn[u][j];
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int n = 0; n < NC; n++) {
            T v = acc[r][n];
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) v = v + __shfl_xor(v, off, 64);
            acc[r][n] = v;
        }
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; r++)
            if (row0 + r < M)
#pragma unroll
                for (int n = 0; n < NC; n++) {
                    T* c = C + (row0 + r) * (int64_t)NC + n;
                    *c = OVERWRITE ? acc[r][n] : *c + acc[r][n];
                }
    }
}

// ---- a large matrix times a batch of columns --------------------------------------------------------------------
// C[M,N] = A[M,K] @ B[K,N] with 3 <= N <= 16: one stream over A.  A block owns 16 rows of A, its eight wavefronts an
// eighth of the k range each, and a wavefront multiplies its 16 x (k range) piece of A into 16 columns on the matrix
// core (v_mfma_f32_16x16x4_f32, v_mfma_f64_16x16x4_f64): lane (row i, quarter q) loads 16 bytes of row i -- the four
// lanes of a row cover 64 contiguous bytes -- and the elements of B for the same k's with plain loads (a step's piece
// of B is 16 x VEC rows of N columns, contiguous, and stays in the caches: B is K x N, a few hundred KiB).  Multiply-add
// e of a step takes element e of every lane, i.e. k = k0 + VEC q + e for q = 0..3: any assignment of k's to the four
// slots of the instruction works as long as A and B use the same one.  Columns from N on are fed zeros.  Nothing
// goes through LDS until the eight partial 16 x 16 results meet there, in wavefront order, at the end: no barrier per
// trip, which is what held the kernel this replaces (B staged through LDS, a barrier per 256 k's) at 33 us for
// [4096,4096] @ [4096,16].
template <typename T> struct Mfma16;
template <> struct Mfma16<float> {
    typedef float Acc __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ Acc mma(float a, float b, Acc c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ int row_of(int q, int v) { return 4 * q + v; }      // accumulator v of lane quarter q
};
template <> struct Mfma16<double> {
    typedef double Acc __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ Acc mma(double a, double b, Acc c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ int row_of(int q, int v) { return 4 * v + q; }
};
template <typename T, bool OVERWRITE>
__global__ __launch_bounds__(512) void matmul_some_cols_kernel(int M, int K, int N, const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C) {
    constexpr int VEC = 16 / (int)sizeof(T);
    constexpr int STEP = 4 * VEC;                                       // k's per step of a wavefront
    constexpr int NW = 8, AHEAD = 4;                                    // wavefronts per block; steps requested together
    typedef T Vec __attribute__((ext_vector_type(VEC)));
    typedef typename Mfma16<T>::Acc Acc;
    __shared__ T part[NW][16][17];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int i = lane & 15, q = lane >> 4;
    const int64_t row0 = (int64_t)blockIdx.x * 16;
    const T* row = A + (row0 + i < M ? row0 + i : M - 1) * (int64_t)K;
    const int steps = (K + STEP - 1) / STEP, per = (steps + NW - 1) / NW;
    const int s0 = wave * per, s1 = s0 + per < steps ? s0 + per : steps;
    const bool col_live = i < N;
    Acc acc = {T(0), T(0), T(0), T(0)};
    // K % VEC == 0 (the host checks): a lane's VEC k's are inside the matrix or all outside
    auto request = [&](Vec (&a)[AHEAD], T (&b)[AHEAD][VEC], int s) {
#pragma unroll
        for (int u = 0; u < AHEAD; u++) {
            const int k = (s + u) * STEP + q * VEC;
            const bool in = s + u < s1 && k < K;
            a[u] = in ? *(const Vec*)(row + k) : Vec(T(0));
#pragma unroll
            for (int e = 0; e < VEC; e++) b[u][e] = (in && col_live) ? B[(int64_t)(k + e) * N + i] : T(0);
        }
    };
    // the next AHEAD steps are on their way while these are multiplied in
    Vec a[AHEAD], an[AHEAD];
    T b[AHEAD][VEC], bn[AHEAD][VEC];
    request(a, b, s0);
    for (int s = s0; s < s1; s += AHEAD) {
        request(an, bn, s + AHEAD);                                     // (past the end: zeros, no memory access)
#pragma unroll
        for (int u = 0; u < AHEAD; u++)
#pragma unroll
            for (int e = 0; e < VEC; e++) acc = Mfma16<T>::mma(a[u][e], b[u][e], acc);
#pragma unroll
        for (int u = 0; u < AHEAD; u++) {
            a[u] = an[u];
#pragma unroll
            for (int e = 0; e < VEC; e++) b[u][e] = bn[u][e];
        }
    }
#pragma unroll
    for (int v = 0; v < 4; v++) part[wave][Mfma16<T>::row_of(q, v)][i] = acc[v];
    __syncthreads();
    if (threadIdx.x < 256) {
        const int r = threadIdx.x >> 4, c = threadIdx.x & 15;
        if (row0 + r < M && c < N) {
            T sum = part[0][r][c];
#pragma unroll
            for (int w = 1; w < NW; w++) sum = sum + part[w][r][c];     // wavefronts in order
            T* dst = C + (row0 + r) * (int64_t)N + c;
            *dst = OVERWRITE ? sum : *dst + sum;
        }
    }
}

// ---- five to 32 rows times a large matrix, on the matrix cores ----------------------------------------------------------
// The same product as matmul_few_rows_kernel computes, C[M,N] = A[M,K] @ B[K,N] with one stream over B, for 5 <= M <= 32:
// with 16 or 32 rows a lane of that kernel issues 64 or 128 multiply-adds per 16 bytes of B, and the vector unit, not the
// stream, sets the pace ([16,4096] @ [4096,4096]: 19 us for 64 MiB).  Here a wavefront owns 16 x VEC columns and
// multiplies its k range into them as 16 x 16 x 4 matrix instructions: lane (j, q) loads 16 bytes of row k0 + VEC q + e'
// of B -- the sixteen lanes j cover 256 contiguous bytes of that row -- and element e of the load belongs to column
// 4 j + e, i.e. to accumulator e; the A operand of the instruction is A[i][k0 + VEC q + e'] out of the block's staged
// piece of A (lane (i, q), one 16-byte LDS read per step).  The four wavefronts of a block sit side by side on 64 x VEC
// columns and walk the same part of the k range, so they never meet; partial rows go to P[part] and
// matmul_add_parts_kernel adds the parts in order.  RG: groups of 16 rows (1 or 2).
template <typename T, int RG>
__global__ __launch_bounds__(256) void matmul_few_rows_mfma_kernel(int M, int K, int N, int k_per_part, int col_blocks, const T* __restrict__ A,
                                                                   const T* __restrict__ B, T* __restrict__ P) {
    constexpr int VEC = 16 / (int)sizeof(T);
    constexpr int STEP = 4 * VEC;                                       // k's per step
    constexpr int KP = 256, AP = KP + VEC;                              // k's a block stages of A; row pitch in LDS
    constexpr int AHEAD = 4;                                            // steps whose rows of B are requested together
    typedef T Vec __attribute__((ext_vector_type(VEC)));
    typedef typename Mfma16<T>::Acc Acc;
    __shared__ __attribute__((aligned(16))) T As[RG * 16][AP];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int j = lane & 15, q = lane >> 4;
    const int part = (int)(blockIdx.x / (unsigned)col_blocks), col_block = (int)(blockIdx.x % (unsigned)col_blocks);
    const int64_t col0 = (((int64_t)col_block * 4 + wave) * 16 + j) * VEC;     // N % VEC == 0 (the host checks)
    const bool live = col0 < N;
    const int k_begin = part * k_per_part;
    const int k_count = k_begin + k_per_part < K ? k_per_part : K - k_begin;     // 1 ... KP
    for (int idx = threadIdx.x; idx < RG * 16 * KP; idx += 256) {
        const int m = idx / KP, kk = idx % KP;
        As[m][kk] = (m < M && kk < k_count) ? A[(int64_t)m * K + k_begin + kk] : T(0);
    }
    Acc acc[RG][VEC];
#pragma unroll
    for (int g = 0; g < RG; g++)
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[g][e] = Acc{T(0), T(0), T(0), T(0)};
    const T* Bc = B + (live ? col0 : 0) + (int64_t)k_begin * N;
    const int steps = (k_count + STEP - 1) / STEP;
    __syncthreads();                                                    // the staged piece of A is complete
    // (requesting the next AHEAD steps while these are multiplied in changed nothing here: 21.4 against 22.7 us for 16 rows)
    for (int s = 0; s < steps; s += AHEAD) {
        Vec b[AHEAD][VEC];
#pragma unroll
        for (int u = 0; u < AHEAD; u++)
#pragma unroll
            for (int r = 0; r < VEC; r++) {
                const int kk = (s + u) * STEP + VEC * q + r;
                b[u][r] = (live && kk < k_count) ? *(const Vec*)(Bc + (int64_t)kk * N) : Vec(T(0));
            }
#pragma unroll
        for (int u = 0; u < AHEAD; u++) {
            if (s + u < steps) {                                        // (uniform; past the end b is zero anyway, this saves the LDS reads)
#pragma unroll
                for (int g = 0; g < RG; g++) {
                    const Vec a = *(const Vec*)&As[16 * g + j][(s + u) * STEP + VEC * q];
#pragma unroll
                    for (int r = 0; r < VEC; r++)
#pragma unroll
                        for (int e = 0; e < VEC; e++) acc[g][e] = Mfma16<T>::mma(a[r], b[u][r][e], acc[g][e]);
                }
            }
        }
    }
    if (live) {
        T* Pp = P + (int64_t)part * M * N + col0;
#pragma unroll
        for (int g = 0; g < RG; g++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int row = 16 * g + Mfma16<T>::row_of(q, v);
                if (row < M) {
                    Vec out;
#pragma unroll
                    for (int e = 0; e < VEC; e++) out[e] = acc[g][e][v];
                    *(Vec*)(Pp + (int64_t)row * N) = out;
                }
            }
    }
}

// The same product where A's rows are whole 16-byte vectors (K a multiple of the vector, A aligned): nothing is staged.
// A block of eight wavefronts owns 16 x VEC columns and a part of the k range; the wavefronts split that part, each
// streams its rows of B as above and reads its piece of A straight from memory (one more 16-byte load per lane, group of
// rows and step: A is a few hundred kilobytes that live in the L2), and they meet once, at the end, in LDS, where the
// first wavefront adds the eight accumulators in order.  With one part the block writes C itself (MODE 1: C = sum,
// 2: C += sum) and the product is one launch; with more (MODE 0) the partial rows go to P[part] as before.
// [16,4096] @ [4096,4096]: 64 column blocks x 4 parts, 16.7 us with the addition of the parts (the staged kernel above:
// 21.2); one part (64 blocks): 31.5, two: 21.3, eight: 17.2.  32 rows: 22.5 (28.8); f64, 16 rows: 24.7 (31.6).
constexpr int FEW_NW = 8;
template <typename T, int RG, int MODE>
__global__ __launch_bounds__(64 * FEW_NW) void matmul_few_rows_split_kernel(int M, int K, int N, int k_per_part, int col_blocks, const T* __restrict__ A,
                                                                           const T* __restrict__ B, T* __restrict__ P) {
    constexpr int VEC = 16 / (int)sizeof(T);
    constexpr int STEP = 4 * VEC;                                       // k's per step
    constexpr int AHEAD = 2;                                            // steps whose rows of B are requested together
    constexpr int PITCH = 16 * VEC + VEC;
    typedef T Vec __attribute__((ext_vector_type(VEC)));
    typedef typename Mfma16<T>::Acc Acc;
    __shared__ __attribute__((aligned(16))) T meet[FEW_NW - 1][RG * 16][PITCH];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int j = lane & 15, q = lane >> 4;
    const int part = (int)(blockIdx.x / (unsigned)col_blocks), col_block = (int)(blockIdx.x % (unsigned)col_blocks);
    const int64_t col0 = ((int64_t)col_block * 16 + j) * VEC;           // N % VEC == 0 (the host checks)
    const bool live = col0 < N;
    const int k_begin = part * k_per_part;
    const int k_end = k_begin + k_per_part < K ? k_begin + k_per_part : K;
    const int steps = (k_end - k_begin + STEP - 1) / STEP;
    const int per_wave = (steps + FEW_NW - 1) / FEW_NW;
    const int s_begin = wave * per_wave, s_end = s_begin + per_wave < steps ? s_begin + per_wave : steps;
    Acc acc[RG][VEC];
#pragma unroll
    for (int g = 0; g < RG; g++)
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[g][e] = Acc{T(0), T(0), T(0), T(0)};
    const T* Bc = B + (live ? col0 : 0);
    Vec b[2][AHEAD][VEC], a[2][AHEAD][RG];
    auto request = [&](int s, Vec (&bb)[AHEAD][VEC], Vec (&aa)[AHEAD][RG]) {
#pragma unroll
        for (int u = 0; u < AHEAD; u++) {
            const int k0 = k_begin + (s + u) * STEP + VEC * q;          // this lane's k's of step s + u: k0 ... k0 + VEC - 1
            const bool step_live = s + u < s_end;
#pragma unroll
            for (int r = 0; r < VEC; r++)
                bb[u][r] = (live && step_live && k0 + r < k_end) ? *(const Vec*)(Bc + (int64_t)(k0 + r) * N) : Vec(T(0));
#pragma unroll
            for (int g = 0; g < RG; g++)                                // (k0 < k_end: the whole vector is, K being a multiple of VEC)
                aa[u][g] = (16 * g + j < M && step_live && k0 < k_end) ? *(const Vec*)(A + (int64_t)(16 * g + j) * K + k0) : Vec(T(0));
        }
    };
    auto multiply = [&](const Vec (&bb)[AHEAD][VEC], const Vec (&aa)[AHEAD][RG]) {
#pragma unroll
        for (int u = 0; u < AHEAD; u++)
#pragma unroll
            for (int g = 0; g < RG; g++)
#pragma unroll
                for (int r = 0; r < VEC; r++)
#pragma unroll
                    for (int e = 0; e < VEC; e++) acc[g][e] = Mfma16<T>::mma(aa[u][g][r], bb[u][r][e], acc[g][e]);
    };
    // two sets of registers: the next AHEAD steps are on their way while these are multiplied in ([16,4096] @ [4096,4096]:
    // 16.7 us; four steps at a time in one set 17.0, eight 17.7, four in two sets 19.0)
    request(s_begin, b[0], a[0]);
    for (int s = s_begin; s < s_end; s += 2 * AHEAD) {
        request(s + AHEAD, b[1], a[1]);
        multiply(b[0], a[0]);
        request(s + 2 * AHEAD, b[0], a[0]);
        multiply(b[1], a[1]);
    }
    if (wave > 0) {
#pragma unroll
        for (int g = 0; g < RG; g++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                Vec out;
#pragma unroll
                for (int e = 0; e < VEC; e++) out[e] = acc[g][e][v];
                *(Vec*)&meet[wave - 1][16 * g + Mfma16<T>::row_of(q, v)][j * VEC] = out;
            }
    }
    __syncthreads();
    if (wave == 0 && live) {
        T* Pp = P + (MODE == 0 ? (int64_t)part * M * N : (int64_t)0) + col0;
#pragma unroll
        for (int g = 0; g < RG; g++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int row = 16 * g + Mfma16<T>::row_of(q, v);
                if (row < M) {
                    Vec sum;
#pragma unroll
                    for (int e = 0; e < VEC; e++) sum[e] = acc[g][e][v];
#pragma unroll
                    for (int w = 0; w < FEW_NW - 1; w++) sum = sum + *(const Vec*)&meet[w][row][j * VEC];     // wavefronts in order
                    Vec* dst = (Vec*)(Pp + (int64_t)row * N);
                    *dst = MODE == 2 ? *dst + sum : sum;
                }
            }
    }
}

// ---- a short inner dimension ------------------------------------------------------------------------------------
// C[M,N] (+)= A[M,K] @ B[K,N] with K <= 16 (the gradient of a weight matrix from a small batch: a sum of K outer
// products): the product writes C once and is bound by that stream.  A thread owns 16 bytes of columns and keeps its
// K x 16 bytes of B in registers; a block walks FEW_RB rows of A, staged in LDS (padded to KC with -0), and writes one
// row of its 256 x 16 bytes of columns per step -- four contiguous kilobytes.
constexpr int FEW_RB = 32;
template <typename T, int KC, bool OVERWRITE>
__global__ __launch_bounds__(256) void matmul_short_inner_kernel(int M, int K, int N, int col_blocks, const T* __restrict__ A,
                                                                 const T* __restrict__ B, T* __restrict__ C) {
    constexpr int VEC = 16 / (int)sizeof(T);
    typedef T Vec __attribute__((ext_vector_type(VEC)));
    typedef T Quad __attribute__((ext_vector_type(4)));
    static_assert(KC % 4 == 0, "the staged rows of A are read four elements at a time");
    __shared__ __attribute__((aligned(16))) T As[FEW_RB][KC];
    const int row_block = (int)(blockIdx.x / (unsigned)col_blocks), col_block = (int)(blockIdx.x % (unsigned)col_blocks);
    const int64_t row0 = (int64_t)row_block * FEW_RB;
    const int64_t col0 = ((int64_t)col_block * 256 + threadIdx.x) * VEC;     // N % VEC == 0 (the host checks)
    const bool live = col0 < N;
    for (int i = threadIdx.x; i < FEW_RB * KC; i += 256) {
        const int r = i / KC, k = i % KC;
        As[r][k] = (k < K && row0 + r < M) ? A[(row0 + r) * K + k] : T(-0.0);     // the padding: products of -0, see below
    }
    Vec b[KC];
#pragma unroll
    for (int k = 0; k < KC; k++) b[k] = (live && k < K) ? *(const Vec*)(B + (int64_t)k * N + col0) : Vec(T(0));
    __syncthreads();
    if (!live) return;
    const int rows = M - row0 < FEW_RB ? (int)(M - row0) : FEW_RB;
    T* Cp = C + row0 * N + col0;
    constexpr int RU = 4;                                               // rows in flight (their old values, when they are read)
    for (int r0 = 0; r0 < rows; r0 += RU) {
        Vec old[RU];
        if (!OVERWRITE) {
#pragma unroll
            for (int u = 0; u < RU; u++) old[u] = *(const Vec*)(Cp + (int64_t)(r0 + u < rows ? r0 + u : rows - 1) * N);
        }
#pragma unroll
        for (int u = 0; u < RU; u++) {
            if (r0 + u < rows) {
                // the reference's own order and rounding (GEMM.java:282-304): the old value, then one rounded product after the
                // other in k order -- the same bits as the simple kernel gives, wherever the operands happen to lie.  The terms
                // beyond K are (-0) x (+0) = -0, and adding -0 changes no float, a zero of either sign included: the loop needs
                // no test on k (with one, sixteen scalar branches per row: 24.9 against 14 us for [4096,16] @ [16,4096]).
                Vec acc = OVERWRITE ? Vec(T(0)) : old[u];
#pragma unroll
                for (int q = 0; q < KC; q += 4) {
                    const Quad a = *(const Quad*)&As[r0 + u][q];
#pragma unroll
                    for (int j = 0; j < 4; j++)
#pragma unroll
                        for (int e = 0; e < VEC; e++) { const T prod = a[j] * b[q + j][e]; acc[e] = acc[e] + prod; }
                }
                *(Vec*)(Cp + (int64_t)(r0 + u) * N) = acc;
            }
        }
    }
}

// ---- f64 on the matrix cores ----------------------------------------------------------------------------------
// 128x128 block tile, four wavefronts in a 2x2 arrangement, each owning 64x64 as 4x4 accumulators of
// v_mfma_f64_16x16x4_f64 (register v of lane l holds row 4*v + l/16 of column l%16 of a 16x16 tile; it feeds A[row l%16]
// [k l/16] and B[k l/16][column l%16]).  k-slices of 16 in double-buffered LDS.
typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));
namespace d64 {
constexpr int DK = 16;
// (pitches: the LDS serves a 64-bit read of 32 lanes per cycle from 64 banks of four bytes, and with these pitches half of
// the passes take a second cycle.  Pitches without any conflict, 18 and BN + 16 (counted: none), measured slower in this
// kernel, 3072^3 892 against 845 us: the LDS is not what bounds it, and two blocks then hold 144 of the unit's 160 KiB.)
constexpr int DA_PITCH = DK + 1;
constexpr int DB_PITCH = BN + 2;
constexpr int LDS_DOUBLES = 2 * BM * DA_PITCH + 2 * DK * DB_PITCH;
}

template <bool EDGE, bool SPLIT = false>
__global__ __launch_bounds__(256, 2) void matmul_mfma_f64_kernel(MfmaArgs g, const double* __restrict__ A,
                                                              const double* __restrict__ B, double* __restrict__ C, double* __restrict__ P = nullptr) {
    using namespace d64;
    __shared__ __attribute__((aligned(16))) double lds[LDS_DOUBLES];
    double* const As0 = lds;                                   // [2][BM * DA_PITCH]
    double* const Bs0 = lds + 2 * BM * DA_PITCH;                // [2][DK * DB_PITCH]
    int tm, tn;
    const int n_tiles = g.tiles_m * g.tiles_n;
    const int part = SPLIT ? (int)blockIdx.x / n_tiles : 0;
    tile_of_block(g, SPLIT ? (int)blockIdx.x - part * n_tiles : (int)blockIdx.x, tm, tn);
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
    const int l16 = lane & 15, q = lane >> 4;

    // global -> registers: A slice 128x16 and B slice 16x128, four 16-byte pieces each per thread
    const int a_row = tid >> 3, a_col = (tid & 7) * 2;       // rows a_row + 32*i
    const int b_row = tid >> 6, b_col = (tid & 63) * 2;      // rows b_row + 4*i
    f64x2 ra[4], rb[4];
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    // A lane's byte offsets inside a slice are fixed for the k loop; the slice moves the base of two buffer descriptors
    // (scalar arithmetic instead of a 64-bit vector addition per load).  EDGE: offsets from the first element of the
    // matrices with the rows past the edge clamped, descriptors that end where the matrices end (k rows of B past the
    // end read as 0); whole tiles: offsets from the tile's first row and column.
    unsigned off_a[4], off_b[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int row = tm * BM + a_row + 32 * i;
        if (EDGE && row > g.M - 1) row = g.M - 1;
        off_a[i] = (unsigned)(row * g.K + a_col) * 8u;
        off_b[i] = (unsigned)((b_row + 4 * i) * g.N + tn * BN + b_col) * 8u;
    }
    auto load_global = [&](int k0) {
        const __amdgpu_buffer_rsrc_t da = __builtin_amdgcn_make_buffer_rsrc((void*)(A + k0), 0, EDGE ? (unsigned)(((int64_t)g.M * g.K - k0) * 8) : 0xffffffffu, 0x00020000);
        const __amdgpu_buffer_rsrc_t db = __builtin_amdgcn_make_buffer_rsrc((void*)(B + (int64_t)k0 * g.N), 0, EDGE ? (unsigned)((int64_t)(g.K - k0) * g.N * 8) : 0xffffffffu, 0x00020000);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            ra[i] = __builtin_bit_cast(f64x2, (u32x4)__builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(da, off_a[i], 0, 0)));
            rb[i] = __builtin_bit_cast(f64x2, (u32x4)__builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(db, off_b[i], 0, 0)));
        }
    };
    // k0: the slice the staging registers hold; its k tail is zeroed here, a slice after the request, and only in the one
    // slice that has a tail (zeroed at the request, every slice would wait for its loads there)
    auto store_lds = [&](int buf, int k0) {
        if (EDGE && k0 + DK > g.K) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
#pragma unroll
                for (int e = 0; e < 2; e++) if (k0 + a_col + e >= g.K) ra[i][e] = 0.0;
                if (k0 + b_row + 4 * i >= g.K) rb[i] = f64x2{0.0, 0.0};
            }
        }
        double* as = As0 + buf * (BM * DA_PITCH);
        double* bs = Bs0 + buf * (DK * DB_PITCH);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            as[(a_row + 32 * i) * DA_PITCH + a_col] = ra[i][0];
            as[(a_row + 32 * i) * DA_PITCH + a_col + 1] = ra[i][1];
            *(f64x2*)(&bs[(b_row + 4 * i) * DB_PITCH + b_col]) = rb[i];
        }
    };

    f64x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = f64x4{0.0, 0.0, 0.0, 0.0};

    const int all_slices = (g.K + DK - 1) / DK;
    const int slice0 = SPLIT ? part * g.split_slices : 0;
    int nk = all_slices;
    if (SPLIT) { nk = all_slices - slice0; if (nk > g.split_slices) nk = g.split_slices; }
    const int kbase = slice0 * DK;
    // Software pipeline over the k-slices, as in the f32 kernels: while the matrix cores work on chunk c (depth 4, sixteen
    // multiply-adds) the operands of chunk c + 1 are read from LDS -- behind the first multiply-adds of the chunk, pinned
    // with scheduling groups, or the compiler sinks the reads behind all sixteen; the next slice, requested at the top of
    // the slice, is written to the other LDS buffer before the last chunk's multiply-adds, and the barrier sits there
    // too, so that the first chunk of the next slice is read under them and no slice begins by waiting for LDS.
    static_assert(DK == 16, "the pipeline below is written for four depth-4 chunks per slice");
    struct Frag64 { double a[4], b[4]; };
    auto read_frag = [&](Frag64& f, int buf, int c) {
        const double* as = As0 + buf * (BM * DA_PITCH);
        const double* bs = Bs0 + buf * (DK * DB_PITCH);
#pragma unroll
        for (int i = 0; i < 4; i++) f.a[i] = as[(wm + 16 * i + l16) * DA_PITCH + 4 * c + q];
#pragma unroll
        for (int j = 0; j < 4; j++) f.b[j] = bs[(4 * c + q) * DB_PITCH + wn + 16 * j + l16];
    };
    auto mma = [&](const Frag64& f) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(f.a[i], f.b[j], acc[i][j], 0, 0, 0);
    };
#define NK_D_MFMA(n) __builtin_amdgcn_sched_group_barrier(0x008, n, 0)
#define NK_D_READ(n) __builtin_amdgcn_sched_group_barrier(0x100, n, 0)
#define NK_D_CHUNK NK_D_MFMA(1); NK_D_READ(2); NK_D_MFMA(1); NK_D_READ(2); NK_D_MFMA(1); NK_D_READ(2); NK_D_MFMA(1); NK_D_READ(2); NK_D_MFMA(12); __builtin_amdgcn_sched_barrier(0)
    Frag64 f0, f1;
    load_global(kbase);
    store_lds(0, kbase);
    __syncthreads();
    read_frag(f0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    for (int kt = 0; kt < nk; kt++) {
        const int cur = kt & 1;
        const bool more = kt + 1 < nk;
        if (more) load_global(kbase + (kt + 1) * DK);
        read_frag(f1, cur, 1);
        mma(f0);
        NK_D_CHUNK;
        read_frag(f0, cur, 2);
        mma(f1);
        NK_D_CHUNK;
        read_frag(f1, cur, 3);
        mma(f0);
        NK_D_CHUNK;
        if (more) {
            store_lds(cur ^ 1, kbase + (kt + 1) * DK);
            __syncthreads();
            read_frag(f0, cur ^ 1, 0);
        }
        mma(f1);
        __builtin_amdgcn_sched_barrier(0);
    }
#undef NK_D_CHUNK
#undef NK_D_READ
#undef NK_D_MFMA

    // epilogue: C is accumulated into; a quarter-wavefront covers 16 consecutive doubles of a row
    const int rows = g.M - tm * BM, cols = g.N - tn * BN;
    double* Cg = (SPLIT ? P + (int64_t)part * g.M * g.N : C) + (int64_t)tm * BM * g.N + tn * BN;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int row = wm + 16 * i + 4 * v + q, col = wn + 16 * j + l16;
                if (!EDGE || (row < rows && col < cols)) {
                    double* p = Cg + (int64_t)row * g.N + col;
                    *p = (SPLIT || g.overwrite) ? acc[i][j][v] : *p + acc[i][j][v];
                }
            }
}

// 64 x 64 block tiles in f64, for the products the f32 kernel of that tile size serves (few large tiles, a last round of large
// tiles that would idle most units, narrow results, long k ranges over few tiles): four wavefronts in a 2 x 2 arrangement,
// each owning 32 x 32 as 2 x 2 accumulators of v_mfma_f64_16x16x4_f64; k-slices of 16 in three LDS stages with the pitches
// of the large kernel.  A multiply-add keeps the matrix core busy for 64 cycles, so the four LDS reads of a depth-4 chunk hide
// behind the multiply-adds of the chunk before it with a single wavefront per SIMD.  EDGE and MIXED as in matmul_mfma64_kernel.
namespace t64d {
constexpr int DK = d64::DK;
// (pitches without bank conflicts: the LDS serves a 64-bit read of 32 lanes per cycle from 64 banks of four bytes.  The 32 lanes
// of a pass read A[row l % 16][k q, q + 1]: with a pitch of 18 doubles the rows fall on the even pairs of banks and the second k
// beside them; B's two k rows of 16 consecutive doubles must lie 32 banks apart: a pitch of 16 modulo 32)
constexpr int A_P = DK + 2, B_P = t64::TN + 16;
constexpr int STAGE = t64::TM * A_P + DK * B_P;
constexpr int LDS_DOUBLES = 3 * STAGE;
}
// (launch bounds of two blocks per unit: with a budget of at most 256 registers the compiler keeps the accumulators in
// ordinary registers; with 512 it moved three of the four between the two register files in every slice, behind a wait for
// the last multiply-add: 0.71 us per slice instead of 0.43 of multiply-adds)
template <bool OVERWRITE, bool EDGE = false, bool MIXED = false>
__global__ __launch_bounds__(256, 2) void matmul_mfma64_f64_kernel(MfmaArgs g, const double* __restrict__ A, const double* __restrict__ B,
                                                                double* __restrict__ C, double* __restrict__ P = nullptr) {
    using namespace t64d;
    constexpr int TM = t64::TM, TN = t64::TN;
    __shared__ __attribute__((aligned(16))) double lds[LDS_DOUBLES];
    int tm, tn, part = 0;
    bool parted = false;
    small_tile_of_block<MIXED>(g, tm, tn, part, parted);
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
    const int l16 = lane & 15, q = lane >> 4;
    // global -> registers: A slice 64 x 16 and B slice 16 x 64, two 16-byte pieces each per thread; byte offsets from the
    // first element of the matrices, fixed for the k loop (the slice moves the base of the descriptors)
    const int a_row = tid >> 3, a_col = (tid & 7) * 2;       // rows a_row + 32 * i
    const int b_row = tid >> 5, b_col = (tid & 31) * 2;      // rows b_row + 8 * i
    f64x2 ra[2], rb[2];
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    unsigned off_a[2], off_b[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        int row = tm * TM + a_row + 32 * i;
        if (EDGE && row > g.M - 1) row = g.M - 1;
        off_a[i] = (unsigned)(row * g.K + a_col) * 8u;
        off_b[i] = (unsigned)((b_row + 8 * i) * g.N + tn * TN + b_col) * 8u;
    }
    auto load_global = [&](int k0) {
        const __amdgpu_buffer_rsrc_t da = __builtin_amdgcn_make_buffer_rsrc((void*)(A + k0), 0, EDGE ? (unsigned)(((int64_t)g.M * g.K - k0) * 8) : 0xffffffffu, 0x00020000);
        const __amdgpu_buffer_rsrc_t db = __builtin_amdgcn_make_buffer_rsrc((void*)(B + (int64_t)k0 * g.N), 0, EDGE ? (unsigned)((int64_t)(g.K - k0) * g.N * 8) : 0xffffffffu, 0x00020000);
#pragma unroll
        for (int i = 0; i < 2; i++) {
            ra[i] = __builtin_bit_cast(f64x2, (u32x4)__builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(da, off_a[i], 0, 0)));
            rb[i] = __builtin_bit_cast(f64x2, (u32x4)__builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(db, off_b[i], 0, 0)));
        }
    };
    // k0: the slice the staging registers hold (EDGE: its k tail is zeroed here, in the one slice that has it)
    auto store_lds = [&](int stage, int k0) {
        if (EDGE && k0 + DK > g.K) {
#pragma unroll
            for (int i = 0; i < 2; i++) {
#pragma unroll
                for (int e = 0; e < 2; e++) if (k0 + a_col + e >= g.K) ra[i][e] = 0.0;
                if (k0 + b_row + 8 * i >= g.K) rb[i] = f64x2{0.0, 0.0};
            }
        }
        double* as = lds + stage * STAGE;
        double* bs = as + TM * A_P;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            *(f64x2*)(&as[(a_row + 32 * i) * A_P + a_col]) = ra[i];
            *(f64x2*)(&bs[(b_row + 8 * i) * B_P + b_col]) = rb[i];
        }
    };
    // operands of one depth-4 chunk: lane quarter q owns k = 4c + q
    struct Chunk { double a[2], b[2]; };
    auto read_chunk = [&](Chunk& f, int stage, int c) {
        const double* as = lds + stage * STAGE;
        const double* bs = as + TM * A_P;
#pragma unroll
        for (int i = 0; i < 2; i++) f.a[i] = as[(wm + 16 * i + l16) * A_P + 4 * c + q];
#pragma unroll
        for (int j = 0; j < 2; j++) f.b[j] = bs[(4 * c + q) * B_P + wn + 16 * j + l16];
    };
    f64x4 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = f64x4{0.0, 0.0, 0.0, 0.0};
    auto mma = [&](const Chunk& f) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(f.a[i], f.b[j], acc[i][j], 0, 0, 0);
    };
    static_assert(DK == 16, "the pipeline below is written for four depth-4 chunks per slice");
    // Three stages of LDS as in matmul_mfma64_kernel: during slice kt the block writes slice kt + 2 and reads slice kt, and
    // the first chunks of slice kt + 1 are read before the barrier, behind the last multiply-adds of slice kt.
    const int all_slices = (g.K + DK - 1) / DK;
    const int slice0 = parted ? part * g.split_slices : 0;
    int nk = all_slices;
    if (parted) { nk = all_slices - slice0; if (nk > g.split_slices) nk = g.split_slices; }
    auto clamped = [&](int slice) { return (slice0 + (slice < nk ? slice : nk - 1)) * DK; };     // past the end: the last slice again, read by nobody
    load_global(clamped(0));
    store_lds(0, clamped(0));
    load_global(clamped(1));
    store_lds(1, clamped(1));
    load_global(clamped(2));                                  // slice 2 waits in the staging registers
    __syncthreads();
    Chunk f0, f1, f2, f3;
    read_chunk(f0, 0, 0);
    read_chunk(f1, 0, 1);
    int cur = 0;
    for (int kt = 0; kt < nk; kt++) {
        const int next = cur == 2 ? 0 : cur + 1, write = next == 2 ? 0 : next + 1;      // stages of slices kt + 1, kt + 2
        read_chunk(f2, cur, 2);
        read_chunk(f3, cur, 3);
        mma(f0);
        mma(f1);
        // the eight LDS reads of chunks 2 and 3 behind the first four multiply-adds of chunks 0 and 1 ...
        NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(4); NK_FENCE;
        store_lds(write, clamped(kt + 2));
        load_global(clamped(kt + 3));
        read_chunk(f0, next, 0);
        read_chunk(f1, next, 1);
        mma(f2);
        mma(f3);
        // ... one LDS write and one request behind each of the next four, the reads of the next slice behind the last four
        NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1); NK_MFMA(1); NK_DS_WRITE(1); NK_VMEM_READ(1);
        NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_MFMA(1); NK_DS_READ(2); NK_FENCE;
        __syncthreads();
        cur = next;
    }
    // register v of accumulator (i, j) sits at row 16 * i + 4 * v + q, column 16 * j + l16 of the wavefront's 32 x 32 tile;
    // a quarter-wavefront covers 16 consecutive doubles of a row
    double* Cg = C + (int64_t)(tm * TM + wm) * g.N + tn * TN + wn;
    if (parted) Cg = P + ((int64_t)part * (g.M - g.rows_a * TM) + (int64_t)((tm - g.rows_a) * TM + wm)) * g.N + tn * TN + wn;
    const int rows = g.M - (tm * TM + wm), cols = g.N - (tn * TN + wn);        // EDGE: what is left of C from the wavefront's first element
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int row = 16 * i + 4 * v + q, col = 16 * j + l16;
                if (!EDGE || (row < rows && col < cols)) {
                    double* p = Cg + (int64_t)row * g.N + col;
                    *p = (OVERWRITE || parted) ? acc[i][j][v] : *p + acc[i][j][v];
                }
            }
}

template <typename T>
static int launch_simple(Device* dev, int64_t M, int64_t K, int64_t N, bool overwrite, const T* A, const T* B, T* C) {
    dim3 grid((unsigned)((N + 63) / 64), (unsigned)((M + 3) / 4));
    NK_REQUIRE(grid.y <= 65535u * 1024u, "nk_matmul: M too large");
    set_path("simple");
    hipLaunchKernelGGL(matmul_simple_kernel<T>, grid, dim3(256), 0, dev->stream, (int)M, (int)K, (int)N, overwrite ? 1 : 0, A, B, C);
    NK_HIP(hipGetLastError());
    return NK_OK;
}

// Few tiles cannot fill 256 compute units (a 512^3 product has 16, a matrix-vector product a single row of them):
// the k range is then cut into parts until there are about two blocks per unit, each part at least four
// k-slices long; the parts are written to the device workspace and added in order by a second launch.
// (`force_parts` >= 2: the caller has planned the number of parts itself, see the row bands in matmul_rm)
static int split_plan(Device* dev, MfmaArgs& g, int slice, size_t elem_bytes, int force_parts = 0) {
    const int tiles = g.tiles_m * g.tiles_n, cus = dev->props.multiProcessorCount;
    const int slices = (g.K + slice - 1) / slice;
    g.splits = 1; g.split_slices = slices;
    if (force_parts < 2 && (tiles >= cus || slices < 8)) return 1;
    int parts = force_parts;
    if (parts < 2) {
        // The number of parts that finishes first, in units of one k-slice of one tile on a compute unit of its own: the
        // blocks a unit ends up with times the slices of a part, plus what a part costs in writing and re-reading its
        // partial tiles.  (Measured: 1024^3, 64 tiles: 4 parts 69 TFLOP/s, 8 parts 59; 1536^3, 144 tiles: 3 parts 89, 4 parts 81.)
        int most = slices / 4 < 64 ? slices / 4 : 64;
        double best = 0;
        for (int p = 2; p <= most; p++) {
            const double cost = (double)(((int64_t)tiles * p + cus - 1) / cus) * ((slices + p - 1) / p) + 0.75 * p;
            if (parts < 2 || cost < best) { parts = p; best = cost; }
        }
        // ... or no parts at all: with nearly a tile per unit (f32 1920^3, 225 tiles: 115 us whole, 124 in two parts) one round
        // of whole tiles (1.80 us per k-slice + 3.5, f64 2.17 + 4.2, and 7 for the launch) beats the parts (1.93, f64 2.2, per
        // unit of the cost above, and 8 for the second launch)
        const bool f64 = elem_bytes == 8;
        if (parts >= 2 && (f64 ? 2.17 : 1.80) * slices + (f64 ? 4.2 : 3.5) + 7.0 <= (f64 ? 2.2 : 1.93) * best + 8.0) return 1;
    }
    if (parts > slices / 4) parts = slices / 4;
    if (parts > 64) parts = 64;
    // bound the workspace: parts * M * N elements
    while (parts > 1 && (uint64_t)parts * g.M * g.N * elem_bytes > ((uint64_t)1 << 30)) parts--;
    if (parts < 2) return 1;
    g.split_slices = (slices + parts - 1) / parts;
    g.splits = (slices + g.split_slices - 1) / g.split_slices;
    return g.splits;
}

template <typename T, typename Launch>
static int launch_mfma(Device* dev, MfmaArgs& g, int slice, T* Cp, Launch launch, int force_parts = 0) {
    const int tiles = g.tiles_m * g.tiles_n;
    void* ws = nullptr;
    if (split_plan(dev, g, slice, sizeof(T), force_parts) > 1) {
        const int64_t mn = (int64_t)g.M * g.N;
        if (int e = workspace(dev, (uint64_t)g.splits * mn * sizeof(T), &ws)) return e;
        launch(true, dim3((unsigned)(tiles * g.splits)), (T*)ws);
        launch_add_parts<T>(dev, mn, g.splits, g.overwrite, (const T*)ws, Cp);
    } else {
        launch(false, dim3((unsigned)tiles), (T*)nullptr);
    }
    NK_HIP(hipGetLastError());
    return NK_OK;
}

// The plans on 64 x 64 tiles, for both element types (`slice`: the depth of a k-slice, 32 floats or 16 doubles -- a slice of a
// small tile then costs the same in both, as a slice of a large tile does).  `launch(mixed, edge, grid, args, P)` starts the
// kernel.  Returns -1 when another plan should take the product.
// `many`: the product has at least a round of large tiles; the small tiles are then held against the plain launch of the large
// ones in rounds of one tile per unit (2560^3 f32, 400 large tiles = 2 rounds for the work of 1.56); otherwise
// against the k range of the large tiles cut into parts.  `walking`: f32 whole tiles with at most eight k-slices.
struct SmallTileNames { const char *whole, *edge, *whole_split, *edge_split, *whole_mixed, *edge_mixed; };
template <typename T, typename Launch>
static int small_tile_plan(Device* dev, const MfmaArgs& g, int slice, bool many, bool whole_small, bool whole_tiles, bool walking,
                           T* Cp, const SmallTileNames& names, Launch launch, double t_beat = 0.0) {
    const int64_t M = g.M, K = g.K, N = g.N;
    const int64_t cus = dev->props.multiProcessorCount;
    const int64_t large = (int64_t)g.tiles_m * g.tiles_n, small = ((M + t64::TM - 1) / t64::TM) * ((N + t64::TN - 1) / t64::TN);
    // A k-slice of a small tile on a unit, microseconds, measured with uniform random operands (small integers run 5 % faster
    // on the small tiles and so flatter them): f32 0.48-0.54 from box to box with a tile per unit, 0.51 over many rounds
    // (3328^3: 589 us); f64 0.54 with a tile per unit and 0.50 with two blocks on a unit (3328^3: 1136 us).
    constexpr bool F64 = sizeof(T) == 8;
    const double c_small = F64 ? (small <= cus ? 0.54 : 0.50) : (many ? 0.51 : 0.50);
    if (many != (large >= cus)) return -1;
    // (very short k ranges over many whole tiles are the walking blocks' case, measured 10-14 % ahead of the small tiles there)
    if (many && walking && large >= 4 * cus && large % 8 == 0) return -1;
    // By estimates fitted to measurements (microseconds, f32): the small tiles run in rounds of one per unit at 0.48 per
    // k-slice plus 5; the parts cost 1.93 per unit of split_plan's estimate plus 8 for the second launch and the shorter blocks.
    // 1024^3 21 against 29 (measured: 21, 31), 1536 x 256 x 1536 17 against 26 (17, 31), 1024 x 1024 x 3072 51 against 60 (53, 64);
    // the parts win 1152^3 36 against 40 (35, 39), 1792^3 108 against 113 (108, 111), 1280 x 4096 x 1280 116 against 128 (107, 127).
    const int64_t slices = (K + slice - 1) / slice;
    const int small_n = (int)((N + t64::TN - 1) / t64::TN), small_m = (int)((M + t64::TM - 1) / t64::TM);
    // ... or whole rounds of small tiles for the upper tile rows and the rest in parts of the k range, in one launch
    // (MIXED, as for the large tiles): 1536^3, 576 small tiles: 2 rounds + 64 tiles in parts instead of 3 rounds, 76 -> 69 us;
    // 1792^3 109 -> 95; 1500^3 78 -> 70 (estimate: the rounds, the parts' rounds of shorter blocks, + 6 for the second launch)
    int64_t mixed_rows = 0, mixed_parts = 0;
    // (per round of tiles, first fetch and write-back: 0.65 for a small f32 tile, 0.95 for f64, against 3.5 and 4.2 for the large
    // ones -- what decides k ranges of a few slices: 3000 x 64 x 3000 f32 19.6 us in 9 rounds of small tiles, 31 in 3 of large ones)
    const double e_small = F64 ? 0.95 : 0.65, e_large = F64 ? 4.2 : 3.5;
    double t_small = (double)((small + cus - 1) / cus) * (c_small * (double)slices + (many ? e_small : 0.0)) + 5.0;
    const int64_t rounds = small / cus, rows_a = rounds * cus / small_n, tiles_b = small - rows_a * small_n;
    if (rounds >= 1 && tiles_b >= 1 && rows_a < small_m && slices >= 16) {
        // the number of parts that finishes first: the units the whole rounds leave idle take parts from the start (as many
        // in a row as fit into a whole tile's time), the rest of the parts runs in rounds of its own; each part is written
        // and read again (1111^3, 252 whole tiles + 72 in parts: 3 parts = 216 blocks fit into one more round, 4 do not)
        const int64_t idle = rounds * cus - rows_a * small_n, m_b = M - rows_a * t64::TM;
        for (int64_t parts = 2; parts <= slices / 4 && parts <= 64; parts++) {
            const int64_t part_slices = (slices + parts - 1) / parts;
            if ((parts - 1) * part_slices >= slices) continue;                      // the last part would be empty
            int64_t left = tiles_b * parts - idle * parts;                          // (idle: in the last of the whole rounds)
            if (left < 0) left = 0;
            const int64_t part_rounds = (left + cus - 1) / cus;
            const double t_mixed = c_small * ((double)rounds * (double)slices + (double)part_rounds * (double)part_slices)
                                 + (many ? e_small * (double)(rounds + part_rounds) : 0.0) + 5.0 + 6.0
                                 + (double)parts * (double)m_b * (double)N * 2.0 * sizeof(T) / 4.0e6;
            if (t_mixed < t_small && (uint64_t)parts * (uint64_t)m_b * N * sizeof(T) <= ((uint64_t)1 << 30)) {
                t_small = t_mixed; mixed_rows = rows_a; mixed_parts = parts;
            }
        }
    }
    // ... or, with less than a round of small tiles, every tile in parts (no upper rows): more blocks per unit at a time
    // for long k ranges over few tiles, and no columns of padding where the large tiles would be half empty
    if (rounds == 0 && slices >= 16) {
        int64_t best = 0; double t_best = t_small;
        for (int64_t parts = 2; parts <= slices / 4 && parts <= 64; parts++) {
            const int64_t part_slices = (slices + parts - 1) / parts;
            if ((parts - 1) * part_slices >= slices) continue;                  // the last part would be empty
            const double t = c_small * (double)((small * parts + cus - 1) / cus) * (double)part_slices + 5.0 + 6.0
                           + (double)parts * (double)M * (double)N * 2.0 * sizeof(T) / 4.0e6;
            if (t < t_best) { t_best = t; best = parts; }
        }
        if (best > 0 && (uint64_t)best * (uint64_t)M * N * sizeof(T) <= ((uint64_t)1 << 30)) { t_small = t_best; mixed_rows = 0; mixed_parts = best; }
    }
    MfmaArgs trial = g;
    // The large tiles.  f32: 1.80 per k-slice and round of one tile per unit (3840^3: 871 us), in parts 1.93 per unit of
    // split_plan's estimate.  The f64 kernel needs its two blocks per unit: 1.84 per slice for each of a pair, 2.17 for a
    // block alone on its unit (2048^3: 278 us; 3328^3, 676 tiles = 512 + 164: 1207 us), in parts 2.2 (1920^3: 300 us).
    double t_large;
    if (many && F64) {
        const int64_t pairs = large / (2 * cus), rest = large - pairs * 2 * cus;
        t_large = (double)slices * ((double)pairs * 2.0 * 1.84 + (rest == 0 ? 0.0 : rest <= cus ? 2.17 : 2.0 * 1.84))
                + e_large * (double)(2 * pairs + (rest == 0 ? 0 : rest <= cus ? 1 : 2)) + 7.0;
    } else if (many) {
        t_large = (double)((large + cus - 1) / cus) * (1.80 * (double)slices + e_large) + 7.0;
    } else {
        const double rate = F64 ? 2.2 : 1.93;
        // (the 128 x 128 edge kernel stores element by element and pads more: 1500^3 measured 86 in parts for an estimate of 72)
        t_large = split_plan(dev, trial, slice, sizeof(T), 0) > 1
            ? (rate * ((double)(((int64_t)large * trial.splits + cus - 1) / cus) * trial.split_slices + 0.75 * trial.splits) + 8.0) * (whole_tiles ? 1.0 : 1.15)
            : ((F64 ? 2.17 : 1.80) * (double)slices + e_large + 7.0) * (whole_tiles ? 1.0 : 1.05);
    }
    if (t_beat > 0.0 && t_beat < t_large) t_large = t_beat;          // (the estimate of another plan that applies: the row bands)
    if (!(t_small < t_large)) return -1;
    MfmaArgs gs = g;
    gs.tiles_m = small_m; gs.tiles_n = small_n;
    gs.group_rows = gs.tiles_m < 8 ? gs.tiles_m : 8;
    if (mixed_parts > 0) {
        gs.rows_a = (int)mixed_rows;
        gs.split_slices = (int)((slices + mixed_parts - 1) / mixed_parts);
        gs.splits = (int)((slices + gs.split_slices - 1) / gs.split_slices);
        const int64_t m_a = mixed_rows * t64::TM, m_b = M - m_a;
        void* ws = nullptr;
        if (int e = workspace(dev, (uint64_t)gs.splits * m_b * N * sizeof(T), &ws)) return e;
        const unsigned grid = (unsigned)(mixed_rows * small_n + (small - mixed_rows * small_n) * gs.splits);
        launch(true, !whole_small, grid, gs, (T*)ws);
        launch_add_parts<T>(dev, m_b * N, gs.splits, g.overwrite, (const T*)ws, Cp + m_a * N);
        NK_HIP(hipGetLastError());
        set_path(mixed_rows == 0 ? (whole_small ? names.whole_split : names.edge_split) : (whole_small ? names.whole_mixed : names.edge_mixed));
        return NK_OK;
    }
    launch(false, !whole_small, (unsigned)small, gs, (T*)nullptr);
    NK_HIP(hipGetLastError());
    set_path(whole_small ? names.whole : names.edge);
    return NK_OK;
}

// `force_parts`, `bands`: how matmul_rm calls itself for the two row bands described below (callers leave them alone: `bands`
// is true for a caller's product, which may be planned as bands or take one of the streaming kernels, and false for a band)
// The 256 x 256 tiles need more LDS (137 KiB) than a launch gets by default: asked for once per device; a device that does
// not grant it (or has less) keeps to the other plans.  Device::big_tiles: 0 not asked yet, 1 granted, -1 not available.
static bool large_lds(Device* dev) {
    if (dev->big_tiles == 0) {
        dev->big_tiles = -1;
        constexpr int big_bytes = big::LDS_FLOATS * (int)sizeof(float);
        if ((int64_t)dev->props.sharedMemPerBlockOptin >= big_bytes) {
            const void* kernels[4] = {(const void*)matmul_mfma_big_kernel<true, false>, (const void*)matmul_mfma_big_kernel<false, false>,
                                      (const void*)matmul_mfma_big_kernel<true, true>, (const void*)matmul_mfma_big_kernel<false, true>};
            hipError_t attr = hipSuccess;
            for (const void* k : kernels)
                if (attr == hipSuccess) attr = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, big_bytes);
            if (attr == hipSuccess) dev->big_tiles = 1; else (void)hipGetLastError();
        }
    }
    return dev->big_tiles > 0;
}

static int matmul_rm(Device* dev, int dtype, bool overwrite, int64_t M, int64_t K, int64_t N, nk_buf A, nk_buf B, nk_buf C,
                     int force_parts = 0, bool bands = true) {
    constexpr int64_t mfma_from = (int64_t)1 << 24;
    MfmaArgs g{};
    g.M = (int)M; g.K = (int)K; g.N = (int)N;
    g.tiles_m = (int)((M + BM - 1) / BM); g.tiles_n = (int)((N + BN - 1) / BN);
    g.group_rows = g.tiles_m < 8 ? g.tiles_m : 8;
    g.overwrite = overwrite ? 1 : 0;
    // Row bands.  Two blocks of a 128 x 128 kernel live on a compute unit, so a launch runs in rounds of 2 x units
    // tiles, and a last round with few tiles costs a whole tile's time on a machine that is mostly idle (f32 3072^3:
    // 576 tiles = one full round + 64 tiles, 100 TFLOP/s; as bands 119-128).  The product is then computed as two
    // products over row bands of A and C, which are matrices of their own in row-major storage: the upper band holds
    // whole rounds of tiles, the lower band's few tiles cut their k range into parts so that they fill one more, short,
    // round (partial results through the workspace, added in order as for every split product).  Times are in units
    // of one tile's time on a compute unit of its own.  Returns -1 when the product is better off in one piece.
    auto run_bands = [&](int elem_bytes, int64_t slices, const char* path, double* estimate = nullptr) -> int {
        if (!bands) return -1;
        const int64_t cus = dev->props.multiProcessorCount, resident = 2 * cus;
        const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
        if (tiles <= resident || tiles >= 8 * resident) return -1;
        const int64_t rows_a = (tiles / resident) * resident / g.tiles_n;               // whole tile rows of the upper band
        const int64_t tiles_a = rows_a * g.tiles_n, tiles_b = tiles - tiles_a;
        if (rows_a < 1 || tiles_b < 1) return -1;
        int64_t parts = resident / tiles_b;
        if (parts > slices / 4) parts = slices / 4;
        if (parts > 64) parts = 64;
        const int64_t m_a = rows_a * BM, m_b = M - m_a;
        const int64_t per16 = 16 / elem_bytes;                                           // the bands keep the alignment of the whole
        if (parts < 2 || m_b * K * N < mfma_from || (m_a * K) % per16 != 0 || (m_a * N) % per16 != 0) return -1;
        const double now = (double)((tiles + cus - 1) / cus);
        const double part_len = (double)((slices + parts - 1) / parts) / (double)slices;
        const double then = (double)((tiles_a + cus - 1) / cus) + 2.0 * part_len + 0.15;     // + two more launches
        if (then >= 0.95 * now) return -1;
        // (`estimate`: only say what the bands would take, in microseconds: a tile's time on a unit is 1.80 per k-slice + 3.5
        // in f32, 1.84 + 4.2 in f64 with its two blocks per unit, and the two further launches cost 8)
        if (estimate) { *estimate = then * ((elem_bytes == 8 ? 1.84 : 1.80) * (double)slices + (elem_bytes == 8 ? 4.2 : 3.5)) + 15.0; return NK_OK; }
        if (int e = matmul_rm(dev, dtype, overwrite, m_a, K, N, A, B, C, 0, false)) return e;
        if (int e = matmul_rm(dev, dtype, overwrite, m_b, K, N, A + (uint64_t)(m_a * K) * elem_bytes, B, C + (uint64_t)(m_a * N) * elem_bytes, (int)parts, false)) return e;
        set_path(path);
        return NK_OK;
    };
    // a few rows of A (at most 32): one stream over B (from 2^24 multiply-adds on, where the sums are re-ordered anyway)
    if (bands && M <= 32 && M * K * N >= mfma_from) {
        const int eb = dtype == NK_F64 ? 8 : 4, vec = 16 / eb;
        if (N % vec == 0 && B % 16 == 0 && N >= 64 * vec) {
            const int64_t col_blocks = (N + 64 * vec - 1) / (64 * vec);
            // about one block per compute unit, a part at least 32 k rows long (eight per wavefront): long parts spread the
            // staging of A and the meeting of the wavefronts over more trips and leave fewer partial rows to add (against
            // two blocks per unit, [16,4096] @ [4096,4096]: 23.4 against 29.7 us, one row: 14.4 against 15.8, 8192^2: 43 against 48)
            int64_t parts = ((int64_t)dev->props.multiProcessorCount + col_blocks - 1) / col_blocks;
            if (parts > K / 32) parts = K / 32;
            if (parts < 1) parts = 1;
            int k_per_part = (int)((K + parts - 1) / parts);
            const int mr = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : M <= 16 ? 16 : 32;
            const bool on_matrix_cores = M > 4;                         // 5 ... 32 rows: 16 x 16 x 4 matrix instructions
            // ... whose wavefronts split the k range inside the block where A's rows are whole vectors: blocks of 16 x vec
            // columns, as many parts as fill the compute units, none shorter than two rounds of requests per wavefront
            if (on_matrix_cores && K % vec == 0 && A % 16 == 0 && N >= 16 * vec) {
                const int64_t blocks_n = (N + 16 * vec - 1) / (16 * vec);
                int64_t split = (int64_t)dev->props.multiProcessorCount / blocks_n;
                const int64_t shortest = (int64_t)FEW_NW * 4 * vec * 8;          // eight steps per wavefront
                if (split > K / shortest) split = K / shortest;
                if (split < 1) split = 1;
                int kpp = (int)((K + split - 1) / split);
                kpp = (kpp + 4 * vec - 1) / (4 * vec) * (4 * vec);                          // whole steps
                split = (K + kpp - 1) / kpp;
                void* wsp = nullptr;
                if (split > 1 && (uint64_t)split * M * N * eb > ((uint64_t)1 << 30)) split = 0;     // (to the kernels below)
                if (split > 1) if (int e = workspace(dev, (uint64_t)split * M * N * eb, &wsp)) return e;
                if (split >= 1) {
                    const dim3 grid((unsigned)(blocks_n * split));
                    auto go = [&](auto t, auto groups_tag) {
                        using T = decltype(t);
                        constexpr int RG = decltype(groups_tag)::value;
                        if (split == 1) {
                            if (g.overwrite) hipLaunchKernelGGL((matmul_few_rows_split_kernel<T, RG, 1>), grid, dim3(64 * FEW_NW), 0, dev->stream, (int)M, (int)K, (int)N, kpp, (int)blocks_n, (const T*)A, (const T*)B, (T*)C);
                            else             hipLaunchKernelGGL((matmul_few_rows_split_kernel<T, RG, 2>), grid, dim3(64 * FEW_NW), 0, dev->stream, (int)M, (int)K, (int)N, kpp, (int)blocks_n, (const T*)A, (const T*)B, (T*)C);
                        } else {
                            hipLaunchKernelGGL((matmul_few_rows_split_kernel<T, RG, 0>), grid, dim3(64 * FEW_NW), 0, dev->stream, (int)M, (int)K, (int)N, kpp, (int)blocks_n, (const T*)A, (const T*)B, (T*)wsp);
                            launch_add_parts<T>(dev, M * N, (int)split, g.overwrite, (const T*)wsp, (T*)C);
                        }
                    };
                    auto by_groups = [&](auto t) { if (M <= 16) go(t, std::integral_constant<int, 1>{}); else go(t, std::integral_constant<int, 2>{}); };
                    if (dtype == NK_F64) by_groups(double{}); else by_groups(float{});
                    NK_HIP(hipGetLastError());
                    set_path(dtype == NK_F64 ? "few_rows_f64" : "few_rows");
                    return NK_OK;
                }
            }
            const int staged = on_matrix_cores ? 256 : few_kp(mr);
            if (k_per_part > staged) k_per_part = staged;               // what a block stages of A
            parts = (K + k_per_part - 1) / k_per_part;
            void* ws = nullptr;
            // the partial rows stay below the 1 GiB every split plan keeps its workspace under; a product beyond that
            // (32 rows against an inner dimension of tens of thousands) goes to the tile kernels below
            if ((uint64_t)parts * M * N * eb <= ((uint64_t)1 << 30)) {
            if (int e = workspace(dev, (uint64_t)parts * M * N * eb, &ws)) return e;
            const dim3 grid((unsigned)(col_blocks * parts));
            auto launch = [&](auto t, auto rows_tag) {
                using T = decltype(t);
                hipLaunchKernelGGL((matmul_few_rows_kernel<T, decltype(rows_tag)::value>), grid, dim3(256), 0, dev->stream, (int)M, (int)K, (int)N, k_per_part, (int)col_blocks,
                                   (const T*)A, (const T*)B, (T*)ws);
                launch_add_parts<T>(dev, M * N, (int)parts, g.overwrite, (const T*)ws, (T*)C);
            };
            auto launch_mfma = [&](auto t, auto groups_tag) {
                using T = decltype(t);
                hipLaunchKernelGGL((matmul_few_rows_mfma_kernel<T, decltype(groups_tag)::value>), grid, dim3(256), 0, dev->stream, (int)M, (int)K, (int)N, k_per_part, (int)col_blocks,
                                   (const T*)A, (const T*)B, (T*)ws);
                launch_add_parts<T>(dev, M * N, (int)parts, g.overwrite, (const T*)ws, (T*)C);
            };
            auto by_rows = [&](auto t) {
                if (M <= 1) launch(t, std::integral_constant<int, 1>{});
                else if (M <= 2) launch(t, std::integral_constant<int, 2>{});
                else if (M <= 4) launch(t, std::integral_constant<int, 4>{});
                else if (M <= 16) launch_mfma(t, std::integral_constant<int, 1>{});
                else launch_mfma(t, std::integral_constant<int, 2>{});
            };
            if (dtype == NK_F64) by_rows(double{}); else by_rows(float{});
            NK_HIP(hipGetLastError());
            set_path(dtype == NK_F64 ? "few_rows_f64" : "few_rows");
            return NK_OK;
            }
        }
    }
    // a batch of columns (3, 5 ... 16): one stream over A on the matrix cores
    if (bands && N <= 16 && N != 1 && N != 2 && N != 4 && M * K * N >= mfma_from) {
        const int eb = dtype == NK_F64 ? 8 : 4, vec = 16 / eb;
        if (K % vec == 0 && A % 16 == 0 && B % 16 == 0 && M >= 1024) {
            const dim3 grid((unsigned)((M + 15) / 16));
            auto launch = [&](auto t) {
                using T = decltype(t);
                if (overwrite) hipLaunchKernelGGL((matmul_some_cols_kernel<T, true>), grid, dim3(512), 0, dev->stream, (int)M, (int)K, (int)N, (const T*)A, (const T*)B, (T*)C);
                else           hipLaunchKernelGGL((matmul_some_cols_kernel<T, false>), grid, dim3(512), 0, dev->stream, (int)M, (int)K, (int)N, (const T*)A, (const T*)B, (T*)C);
            };
            if (dtype == NK_F64) launch(double{}); else launch(float{});
            NK_HIP(hipGetLastError());
            set_path(dtype == NK_F64 ? "some_cols_f64" : "some_cols");
            return NK_OK;
        }
    }
    // a short inner dimension: one stream over C
    if (bands && K <= 16 && M * K * N >= mfma_from) {
        const int eb = dtype == NK_F64 ? 8 : 4, vec = 16 / eb;
        if (N % vec == 0 && N >= 64 * vec && B % 16 == 0 && C % 16 == 0) {
            const int64_t col_blocks = (N + 256 * vec - 1) / (256 * vec), row_blocks = (M + FEW_RB - 1) / FEW_RB;
            const dim3 grid((unsigned)(col_blocks * row_blocks));
            auto launch = [&](auto t, auto kc) {
                using T = decltype(t);
                constexpr int KC = decltype(kc)::value;
                if (overwrite) hipLaunchKernelGGL((matmul_short_inner_kernel<T, KC, true>), grid, dim3(256), 0, dev->stream, (int)M, (int)K, (int)N, (int)col_blocks, (const T*)A, (const T*)B, (T*)C);
                else           hipLaunchKernelGGL((matmul_short_inner_kernel<T, KC, false>), grid, dim3(256), 0, dev->stream, (int)M, (int)K, (int)N, (int)col_blocks, (const T*)A, (const T*)B, (T*)C);
            };
            auto by_depth = [&](auto t) {
                if (K <= 4) launch(t, std::integral_constant<int, 4>{});
                else if (K <= 8) launch(t, std::integral_constant<int, 8>{});
                else launch(t, std::integral_constant<int, 16>{});
            };
            if (dtype == NK_F64) by_depth(double{}); else by_depth(float{});
            NK_HIP(hipGetLastError());
            set_path(dtype == NK_F64 ? "short_inner_f64" : "short_inner");
            return NK_OK;
        }
        // not aligned, or rows shorter than a wavefront of vectors: the simple kernel, which gives the same bits (a
        // matrix-core plan would re-order sixteen terms for nothing); a few columns have their own plan below
        if (N > 16) return dtype == NK_F64 ? launch_simple<double>(dev, M, K, N, overwrite, (const double*)A, (const double*)B, (double*)C)
                               : launch_simple<float>(dev, M, K, N, overwrite, (const float*)A, (const float*)B, (float*)C);
    }
    // a few columns of B: one stream over A
    if (bands && N <= 4 && M * K * N >= mfma_from) {
        const int eb = dtype == NK_F64 ? 8 : 4, vec = 16 / eb;
        if (K % vec == 0 && A % 16 == 0 && B % 16 == 0 && (N == 1 || N == 2 || N == 4)) {
            auto launch = [&](auto t, auto nc) {
                using T = decltype(t);
                constexpr int NC = decltype(nc)::value;
                // four rows per wavefront while that leaves two blocks per compute unit, else one
                const bool four = (M + 15) / 16 >= 2 * (int64_t)dev->props.multiProcessorCount;
                const unsigned blocks = (unsigned)(four ? (M + 15) / 16 : (M + 3) / 4);
                if (four) {
                    if (overwrite) hipLaunchKernelGGL((matmul_few_cols_kernel<T, NC, 4, true>), dim3(blocks), dim3(256), 0, dev->stream, (int)M, (int)K, (const T*)A, (const T*)B, (T*)C);
                    else           hipLaunchKernelGGL((matmul_few_cols_kernel<T, NC, 4, false>), dim3(blocks), dim3(256), 0, dev->stream, (int)M, (int)K, (const T*)A, (const T*)B, (T*)C);
                } else {
                    if (overwrite) hipLaunchKernelGGL((matmul_few_cols_kernel<T, NC, 1, true>), dim3(blocks), dim3(256), 0, dev->stream, (int)M, (int)K, (const T*)A, (const T*)B, (T*)C);
                    else           hipLaunchKernelGGL((matmul_few_cols_kernel<T, NC, 1, false>), dim3(blocks), dim3(256), 0, dev->stream, (int)M, (int)K, (const T*)A, (const T*)B, (T*)C);
                }
            };
            auto by_cols = [&](auto t) {
                if (N == 1) launch(t, std::integral_constant<int, 1>{});
                else if (N == 2) launch(t, std::integral_constant<int, 2>{});
                else launch(t, std::integral_constant<int, 4>{});
            };
            if (dtype == NK_F64) by_cols(double{}); else by_cols(float{});
            NK_HIP(hipGetLastError());
            set_path(dtype == NK_F64 ? "few_cols_f64" : "few_cols");
            return NK_OK;
        }
    }
    if (dtype == NK_F64) {
        // from 2^24 multiply-adds on the matrix cores take over (sums re-ordered, within 1e-12 of the reference);
        // smaller products keep the reference's summation order bit for bit
        const bool fits = M * K * 8 < ((int64_t)1 << 32) && K * N * 8 < ((int64_t)1 << 32);
        if (M * K * N >= mfma_from && fits) {
            const bool whole = (A % 16 == 0) && (B % 16 == 0) && M % BM == 0 && N % BN == 0 && K % d64::DK == 0;
            const double* Ap = (const double*)A; const double* Bp = (const double*)B; double* Cp = (double*)C;
            // the plans on 64 x 64 tiles, as for f32 below: before the bands for products with less than a round of large tiles,
            // after them for larger ones
            const bool whole_small = (A % 16 == 0) && (B % 16 == 0) && M % t64::TM == 0 && N % t64::TN == 0 && K % d64::DK == 0;
            auto small_tile_plan = [&](bool many, double t_beat = 0.0) -> int {
                if (!(bands && force_parts < 2 && K > 16)) return -1;
                static const SmallTileNames names = {"mfma_f64_tiles_of_64", "mfma_f64_tiles_of_64_edge", "mfma_f64_tiles_of_64_split", "mfma_f64_tiles_of_64_edge_split",
                                                     "mfma_f64_tiles_of_64_mixed", "mfma_f64_tiles_of_64_edge_mixed"};
                return nk::small_tile_plan<double>(dev, g, d64::DK, many, whole_small, whole, false, Cp, names,
                    [&](bool mixed, bool edge_kernel, unsigned grid, const MfmaArgs& gs, double* P) {
                        auto go = [&](auto kernel) { hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), 0, dev->stream, gs, Ap, Bp, Cp, P); };
                        if (mixed) {
                            if (edge_kernel) { if (overwrite) go(matmul_mfma64_f64_kernel<true, true, true>); else go(matmul_mfma64_f64_kernel<false, true, true>); }
                            else             { if (overwrite) go(matmul_mfma64_f64_kernel<true, false, true>); else go(matmul_mfma64_f64_kernel<false, false, true>); }
                        } else {
                            if (edge_kernel) { if (overwrite) go(matmul_mfma64_f64_kernel<true, true, false>); else go(matmul_mfma64_f64_kernel<false, true, false>); }
                            else             { if (overwrite) go(matmul_mfma64_f64_kernel<true, false, false>); else go(matmul_mfma64_f64_kernel<false, false, false>); }
                        }
                    }, t_beat);
            };
            if (const int rc = small_tile_plan(false); rc >= 0) return rc;
            // where the row bands apply, the small tiles must beat them clearly (short k ranges: 3072 x 320 x 3072)
            double t_bands = 0.0;
            const char* bands_name = whole ? "mfma_f64_bands" : "mfma_f64_edge_bands";
            if (run_bands(8, (K + d64::DK - 1) / d64::DK, bands_name, &t_bands) >= 0) {
                if (const int rc = small_tile_plan(true, 0.93 * t_bands); rc >= 0) return rc;
                if (const int rc = run_bands(8, (K + d64::DK - 1) / d64::DK, bands_name); rc >= 0) return rc;
            }
            if (const int rc = small_tile_plan(true); rc >= 0) return rc;
            const int rc = launch_mfma<double>(dev, g, d64::DK, Cp, [&](bool split, dim3 grid, double* P) {
                if (whole && split)       hipLaunchKernelGGL((matmul_mfma_f64_kernel<false, true>), grid, dim3(256), 0, dev->stream, g, Ap, Bp, Cp, P);
                else if (whole)           hipLaunchKernelGGL((matmul_mfma_f64_kernel<false, false>), grid, dim3(256), 0, dev->stream, g, Ap, Bp, Cp, P);
                else if (split)           hipLaunchKernelGGL((matmul_mfma_f64_kernel<true, true>), grid, dim3(256), 0, dev->stream, g, Ap, Bp, Cp, P);
                else                      hipLaunchKernelGGL((matmul_mfma_f64_kernel<true, false>), grid, dim3(256), 0, dev->stream, g, Ap, Bp, Cp, P);
            }, force_parts);
            set_path(whole ? (g.splits > 1 ? "mfma_f64_split" : "mfma_f64") : (g.splits > 1 ? "mfma_f64_edge_split" : "mfma_f64_edge"));
            return rc;
        }
        return launch_simple<double>(dev, M, K, N, overwrite, (const double*)A, (const double*)B, (double*)C);
    }
    const bool aligned = (A % 16 == 0) && (B % 16 == 0) && (C % 16 == 0);
    // (the whole-tile kernels address a slice with 32-bit byte offsets from its first element: 256 rows of A, 32 rows of B)
    const bool whole_tiles = aligned && M % BM == 0 && N % BN == 0 && K % BK == 0 && K < ((int64_t)1 << 20) && N < ((int64_t)1 << 23);
    // Small products stay on the simple kernel, which keeps the reference's summation order bit for bit; from
    // 2^24 multiply-adds on, shapes that are not whole tiles take the matrix cores through the edge variant.
    const bool edge = !whole_tiles && M * K * N >= mfma_from && M * K * 4 < ((int64_t)1 << 32) && K * N * 4 < ((int64_t)1 << 32);
    if (whole_tiles || edge) {
        const float* Ap = (const float*)A; const float* Bp = (const float*)B; float* Cp = (float*)C;
        // 256x256 tiles, one block per compute unit, when they fill the machine in whole rounds (or many rounds) and the
        // tiles are deep enough for the first fetch and the write-back not to weigh: with one block per compute unit
        // nothing overlaps a tile's write-back, and reading the old C as well doubles it (measured on 8192 x K x 8192
        // against the kernels with two blocks per unit -- C = A B: 115 against 112 TFLOP/s at K = 256, 132 against 125
        // at 512; C += A B: 105 against 112, 121 against 126, the same at 768; 65536 x 256 x 256, a single round of
        // tiles: 79 against 73 us)
        if (K >= (overwrite ? 16 : 32) * BK) {
            const bool whole_big = whole_tiles && M % big::TM == 0 && N % big::TN == 0;
            const int64_t cus = dev->props.multiProcessorCount;
            const int64_t tiles = ((M + big::TM - 1) / big::TM) * ((N + big::TN - 1) / big::TN);
            if ((whole_big || edge) && tiles >= cus && (tiles % cus == 0 || tiles >= 4 * cus)) {
                MfmaArgs gb = g;
                gb.tiles_m = (int)((M + big::TM - 1) / big::TM); gb.tiles_n = (int)((N + big::TN - 1) / big::TN);
                gb.group_rows = gb.tiles_m < 4 ? gb.tiles_m : 4;
                constexpr int lds_bytes = big::LDS_FLOATS * (int)sizeof(float);
                large_lds(dev);
                if (dev->big_tiles > 0) {
                    const dim3 grid((unsigned)tiles);
                    if (whole_big) {
                        if (overwrite) hipLaunchKernelGGL((matmul_mfma_big_kernel<true, false>), grid, dim3(256), lds_bytes, dev->stream, gb, Ap, Bp, Cp);
                        else           hipLaunchKernelGGL((matmul_mfma_big_kernel<false, false>), grid, dim3(256), lds_bytes, dev->stream, gb, Ap, Bp, Cp);
                    } else {
                        if (overwrite) hipLaunchKernelGGL((matmul_mfma_big_kernel<true, true>), grid, dim3(256), lds_bytes, dev->stream, gb, Ap, Bp, Cp);
                        else           hipLaunchKernelGGL((matmul_mfma_big_kernel<false, true>), grid, dim3(256), lds_bytes, dev->stream, gb, Ap, Bp, Cp);
                    }
                    NK_HIP(hipGetLastError());
                    set_path(whole_big ? "mfma_big" : "mfma_big_edge");
                    return NK_OK;
                }
            }
        }
        // fewer large tiles than compute units, but whole 64 x 64 tiles, at least one per unit: the small-tile kernel in one launch
        const bool whole_small = aligned && M % t64::TM == 0 && N % t64::TN == 0 && K % BK == 0;
        const bool fits_32_bits = M * K * 4 < ((int64_t)1 << 32) && K * N * 4 < ((int64_t)1 << 32);       // (the edge kernels' offsets)
        auto small_tile_plan = [&](bool many, double t_beat = 0.0) -> int {
            // (from the shortest k ranges on, above the ones of the short-inner kernel: the kernel reads its slices clamped to
            // the last one, and with one or two slices a small tile's fetch and write-back overlap better with the other blocks
            // of its unit -- 3000 x 64 x 3000 31 -> 19 us, 100000 x 64 x 64 31 -> 16, 1000 x 100 x 1000 15 -> 6)
            if (!(bands && force_parts < 2 && (whole_small || fits_32_bits) && K > 16)) return -1;
            static const SmallTileNames names = {"mfma_tiles_of_64", "mfma_tiles_of_64_edge", "mfma_tiles_of_64_split", "mfma_tiles_of_64_edge_split",
                                                 "mfma_tiles_of_64_mixed", "mfma_tiles_of_64_edge_mixed"};
            return nk::small_tile_plan<float>(dev, g, BK, many, whole_small, whole_tiles, whole_tiles && K / BK <= 8, Cp, names,
                [&](bool mixed, bool edge_kernel, unsigned grid, const MfmaArgs& gs, float* P) {
                    auto go = [&](auto kernel) { hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), 0, dev->stream, gs, Ap, Bp, Cp, P); };
                    if (mixed) {
                        if (edge_kernel) { if (overwrite) go(matmul_mfma64_kernel<true, true, true>); else go(matmul_mfma64_kernel<false, true, true>); }
                        else             { if (overwrite) go(matmul_mfma64_kernel<true, false, true>); else go(matmul_mfma64_kernel<false, false, true>); }
                    } else {
                        if (edge_kernel) { if (overwrite) go(matmul_mfma64_kernel<true, true, false>); else go(matmul_mfma64_kernel<false, true, false>); }
                        else             { if (overwrite) go(matmul_mfma64_kernel<true, false, false>); else go(matmul_mfma64_kernel<false, false, false>); }
                    }
                }, t_beat);
        };

        if (const int rc = small_tile_plan(false); rc >= 0) return rc;
        {
            double t_bands = 0.0;
            const char* bands_name = whole_tiles ? "mfma_bands" : "mfma_edge_bands";
            if (run_bands(4, (K + BK - 1) / BK, bands_name, &t_bands) >= 0) {
                if (const int rc = small_tile_plan(true, 0.93 * t_bands); rc >= 0) return rc;
                if (const int rc = run_bands(4, (K + BK - 1) / BK, bands_name); rc >= 0) return rc;
            }
        }
        // A few more tiles than a whole number of rounds of one tile per compute unit: as one launch of whole tiles some units
        // would work through one tile more than the others (side by side with another).  Instead the upper tile rows, whole
        // rounds, take the whole k range, and the tiles of the lower rows come as parts of their k range that fill the
        // gaps (matmul_mfma_kernel<false, false, true>); their sum follows as for every split product.  2304^3 (324 tiles):
        // 278 -> 203 us; 2176 x 2048 x 2176: 247 -> 164; 3584^3 (784): 805 -> 648; 4608^3 (1296): 1549 -> 1353.  With more
        // than half a round of tiles in the lower rows it no longer pays (2560^3, 160 of 400 tiles: 310 -> 302; 4096 x 512 x
        // 1536, 132 of 384: 68 -> 75); where two row bands apply (above) they are level or ahead (3072^3: 414 against 426).
        if (bands && force_parts < 2) {
            const int64_t cus = dev->props.multiProcessorCount, tiles = (int64_t)g.tiles_m * g.tiles_n, slices = (K + BK - 1) / BK;
            const int64_t rounds = tiles / cus;
            const int64_t rows_a = rounds * cus / g.tiles_n;
            const int64_t tiles_b = tiles - rows_a * g.tiles_n;
            if (tiles > cus && rounds >= 1 && rounds <= 6 && tiles_b >= 1 && 2 * tiles_b <= cus && rows_a >= 1 && rows_a < g.tiles_m && slices >= 16) {
                const int64_t m_a = rows_a * BM, m_b = M - m_a;
                int64_t parts = (2 * cus + tiles_b - 1) / tiles_b;                        // about two short blocks per unit at a time
                if (parts > slices / 8) parts = slices / 8;
                if (parts >= 2 && (uint64_t)parts * m_b * N * sizeof(float) <= ((uint64_t)1 << 30)) {
                    MfmaArgs gm = g;
                    gm.rows_a = (int)rows_a;
                    gm.split_slices = (int)((slices + parts - 1) / parts);
                    gm.splits = (int)((slices + gm.split_slices - 1) / gm.split_slices);
                    void* ws = nullptr;
                    if (int e = workspace(dev, (uint64_t)gm.splits * m_b * N * sizeof(float), &ws)) return e;
                    const unsigned grid = (unsigned)(rows_a * g.tiles_n + tiles_b * gm.splits);
                    if (whole_tiles) hipLaunchKernelGGL((matmul_mfma_kernel<false, false, true>), dim3(grid), dim3(256), 0, dev->stream, gm, Ap, Bp, Cp, (float*)ws);
                    else             hipLaunchKernelGGL((matmul_mfma_kernel<true, false, true>), dim3(grid), dim3(256), 0, dev->stream, gm, Ap, Bp, Cp, (float*)ws);
                    launch_add_parts<float>(dev, m_b * N, gm.splits, g.overwrite, (const float*)ws, Cp + m_a * N);
                    NK_HIP(hipGetLastError());
                    set_path(whole_tiles ? "mfma_mixed" : "mfma_edge_mixed");
                    return NK_OK;
                }
            }
        }
        if (const int rc = small_tile_plan(true); rc >= 0) return rc;
        bool streamed = false;
        const int rc = launch_mfma<float>(dev, g, BK, Cp, [&](bool split, dim3 grid, float* P) {
            if (whole_tiles && split) hipLaunchKernelGGL((matmul_mfma_kernel<false, true>), grid, dim3(256), 0, dev->stream, g, Ap, Bp, Cp, P);
            else if (whole_tiles) {
                // more tiles than blocks that fit the machine at one time: the blocks stay and walk the tiles
                const unsigned resident = 2u * (unsigned)dev->props.multiProcessorCount;
                const unsigned tiles = (unsigned)(g.tiles_m * g.tiles_n);
                // (pays while a tile has very few k-slices, i.e. while its first fetch and its write-back weigh: measured
                // +3 % at 8 slices, -3 % at 16 against the tile kernel)
                if (g.K / BK <= 8 && tiles >= 2 * resident && tiles % 8 == 0 && resident % 8 == 0) {
                    if (overwrite) hipLaunchKernelGGL(matmul_mfma_stream_kernel<true>, dim3(resident), dim3(256), 0, dev->stream, g, Ap, Bp, Cp);
                    else           hipLaunchKernelGGL(matmul_mfma_stream_kernel<false>, dim3(resident), dim3(256), 0, dev->stream, g, Ap, Bp, Cp);
                    streamed = true;
                }
                else
                    hipLaunchKernelGGL((matmul_mfma_kernel<false, false>), grid, dim3(256), 0, dev->stream, g, Ap, Bp, Cp, P);
            }
            else if (split)           hipLaunchKernelGGL((matmul_mfma_kernel<true, true>), grid, dim3(256), 0, dev->stream, g, Ap, Bp, Cp, P);
            else                      hipLaunchKernelGGL((matmul_mfma_kernel<true, false>), grid, dim3(256), 0, dev->stream, g, Ap, Bp, Cp, P);
        }, force_parts);
        set_path(streamed ? "mfma_stream" : whole_tiles ? (g.splits > 1 ? "mfma_split" : "mfma") : (g.splits > 1 ? "mfma_edge_split" : "mfma_edge"));
        return rc;
    }
    return launch_simple<float>(dev, M, K, N, overwrite, (const float*)A, (const float*)B, (float*)C);
}

}  // namespace nk

using namespace nk;

static int matmul_entry(nk_dev h, bool overwrite, int dtype, int layout, int64_t M, int64_t K, int64_t N, nk_buf A, nk_buf B, nk_buf C) {
    NK_DEVICE(dev, h);
    NK_REQUIRE(dtype == NK_F32 || dtype == NK_F64, "nk_matmul: unknown dtype %d", dtype);
    NK_REQUIRE(layout == NK_LAYOUT_ROW_MAJOR || layout == NK_LAYOUT_COLUMN_MAJOR, "nk_matmul: unknown layout %d", layout);
    NK_REQUIRE(M >= 1 && K >= 1 && N >= 1, "nk_matmul: M, K, N must be positive (got %lld, %lld, %lld)", (long long)M, (long long)K, (long long)N);
    NK_REQUIRE(M * K < ((int64_t)1 << 31) && K * N < ((int64_t)1 << 31) && M * N < ((int64_t)1 << 31),
               "nk_matmul: operands are limited to 2^31-1 elements");
    const int eb = dtype_bytes(dtype);
    if (int e = check_range(dev, "nk_matmul(A)", A, 0, (uint64_t)(M * K) * eb)) return e;
    if (int e = check_range(dev, "nk_matmul(B)", B, 0, (uint64_t)(K * N) * eb)) return e;
    if (int e = check_range(dev, "nk_matmul(C)", C, 0, (uint64_t)(M * N) * eb)) return e;
    if (layout == NK_LAYOUT_ROW_MAJOR) return matmul_rm(dev, dtype, overwrite, M, K, N, A, B, C);
    // column-major data of X[r,c] is the row-major data of X^T[c,r]:  C^T[N,M] += B^T[N,K] @ A^T[K,M]
    return matmul_rm(dev, dtype, overwrite, N, K, M, B, A, C);
}

extern "C" int nk_matmul(nk_dev h, int dtype, int layout, int64_t M, int64_t K, int64_t N, nk_buf A, nk_buf B, nk_buf C) {
    return matmul_entry(h, false, dtype, layout, M, K, N, A, B, C);
}

extern "C" int nk_matmul_set(nk_dev h, int dtype, int layout, int64_t M, int64_t K, int64_t N, nk_buf A, nk_buf B, nk_buf C) {
    return matmul_entry(h, true, dtype, layout, M, K, N, A, B, C);
}
