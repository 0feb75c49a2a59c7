// nk_sum, nk_reduce_index, nk_dot: whole-tensor reductions of a dense buffer.
//
// The reference's CPU device reduces in a fixed tree: tiles of RTS consecutive elements are reduced front to
// back, the tile results are reduced the same way, until one value is left (CPUSum: RTS = 128, the value starts
// at 0; CPUReduce: RTS = 64, strict comparison, the first winner keeps its place and its index into the
// original data is the result).  J/backend/main/operations/other/internal/CPUSum.java:26-74, CPUReduce.java:90-157.
// The kernels here keep exactly that tree, so sums are bit-identical to the CPU device and min/max return the
// same index, ties and NaNs included.
//
// One level of the tree: a wavefront owns 64 consecutive tiles, i.e. one contiguous piece of memory.  It moves
// the piece through LDS 32 columns at a time -- 16-byte buffer loads that run along memory, rows of 33
// elements in LDS -- and lane t then walks front to back through the 32 values of tile t (conflict-free).  The
// loads of the next 32 columns are in flight while the current ones are reduced.  Elements past the end of the
// data read as zero through the buffer range check and are skipped by the tile's own limit.  A block's 256 tile
// results are whole tiles of the next level (256 = 2 x 128 = 4 x 64), which the block reduces itself: one launch
// covers two levels of the tree.
#include "nk_internal.h"

namespace nk {

typedef __amdgpu_buffer_rsrc_t BufRsrc;
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

enum { STAT_SUM = 0, STAT_MIN = 1, STAT_MAX = 2, STAT_DOT = 3 };

template <typename T, int RTS, int MODE>
__global__ __launch_bounds__(256) void tile_reduce_kernel(const T* __restrict__ in, const T* __restrict__ in2,
                                                          const int* __restrict__ idx_in, int64_t n,
                                                          T* __restrict__ out, int* __restrict__ idx_out, int pieces) {
    constexpr int VEC = 16 / sizeof(T);             // elements per 16-byte load
    constexpr int COLS = 32;                        // columns staged at a time
    constexpr int NCH = RTS / COLS;
    constexpr int LOADS = 64 * COLS / VEC / 64;     // 16-byte loads per lane and chunk
    constexpr int PPR = COLS / VEC;                 // 16-byte pieces per tile row of a chunk
    __shared__ T stage[4][64][COLS + 1];
    constexpr bool INDEXED = MODE == STAT_MIN || MODE == STAT_MAX;
    constexpr int NEXT = 256 / RTS;                  // next-level tiles per piece
    __shared__ __attribute__((aligned(16))) T level_val[256];
    __shared__ int level_idx[INDEXED ? 256 : 1];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    // A block walks `pieces` consecutive pieces of 256 tiles (what used to be one block each): few long-running blocks
    // that each read one contiguous stretch stream faster than many short ones, and the first chunk of the next piece
    // is requested while the last chunk of the current one is reduced.  One buffer descriptor per wavefront spans from
    // its first tile to the end of the data; the piece and the chunk go into the scalar offset of the loads.
    const int64_t piece0 = (int64_t)blockIdx.x * pieces;
    const int64_t wave_elem0 = (piece0 * 4 + wave) * 64 * RTS;           // first element of the wavefront in piece 0
    const int64_t wave_left = wave_elem0 < n ? n - wave_elem0 : 0;       // nothing left: every load reads zeros
    const unsigned bytes = wave_left * (int64_t)sizeof(T) > 0xffffffffll ? 0xffffffffu : (unsigned)(wave_left * sizeof(T));
    const BufRsrc r1 = __builtin_amdgcn_make_buffer_rsrc((void*)(in + (wave_left > 0 ? wave_elem0 : 0)), 0, bytes, 0x00020000);
    const BufRsrc r2 = __builtin_amdgcn_make_buffer_rsrc((void*)((MODE == STAT_DOT ? in2 : in) + (wave_left > 0 ? wave_elem0 : 0)), 0, bytes, 0x00020000);
    T (*mine)[COLS + 1] = stage[wave];

    // piece k of the lane inside a chunk: tile row and column of its 16 bytes
    unsigned voff[LOADS];
    int prow[LOADS], pcol[LOADS];
#pragma unroll
    for (int k = 0; k < LOADS; k++) {
        const int p = lane + 64 * k;
        prow[k] = p / PPR;
        pcol[k] = (p % PPR) * VEC;
        voff[k] = (unsigned)((prow[k] * RTS + pcol[k]) * sizeof(T));
    }
    // one chunk ahead (two in flight measured slower: 47.1 against 45.1 us for the sum of 2^26 floats)
    u32x4 cur[LOADS], cur2[LOADS];
    constexpr int NON_TEMPORAL = 2;                 // cache policy of the loads: every element is read exactly once
    constexpr unsigned PIECE_BYTES = 256u * RTS * sizeof(T);
    auto request = [&](int piece_i, int c) {
        const unsigned soff = (unsigned)piece_i * PIECE_BYTES + (unsigned)(c * COLS * sizeof(T));
#pragma unroll
        for (int k = 0; k < LOADS; k++) {
            cur[k] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r1, voff[k], soff, NON_TEMPORAL));
            if (MODE == STAT_DOT)
                cur2[k] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r2, voff[k], soff, NON_TEMPORAL));
        }
    };
    request(0, 0);
    for (int piece_i = 0; piece_i < pieces; piece_i++) {
    const int64_t piece = piece0 + piece_i;
    const int64_t elem0 = (piece * 4 + wave) * 64 * RTS;

    // the lane's own tile
    const int64_t my_first = elem0 + (int64_t)lane * RTS;
    int limit = 0;
    if (my_first < n) limit = n - my_first < RTS ? (int)(n - my_first) : RTS;
    T value = T(0);
    int found = 0;

#pragma unroll
    for (int c = 0; c < NCH; c++) {
#pragma unroll
        for (int k = 0; k < LOADS; k++) {
            typedef T Vec __attribute__((ext_vector_type(VEC)));
            const Vec v = __builtin_bit_cast(Vec, cur[k]);
            if (MODE == STAT_DOT) {
                const Vec w = __builtin_bit_cast(Vec, cur2[k]);
#pragma unroll
                for (int e = 0; e < VEC; e++) mine[prow[k]][pcol[k] + e] = v[e] * w[e];       // rounded product
            } else {
#pragma unroll
                for (int e = 0; e < VEC; e++) mine[prow[k]][pcol[k] + e] = v[e];
            }
        }
        if (c + 1 < NCH) request(piece_i, c + 1);
        else if (piece_i + 1 < pieces) request(piece_i + 1, 0);
        __builtin_amdgcn_wave_barrier();            // LDS operations of a wavefront complete in order
#pragma unroll
        for (int i = 0; i < COLS; i++) {
            const T x = mine[lane][i];
            const int pos = c * COLS + i;
            if (MODE == STAT_SUM || MODE == STAT_DOT) {
                if (pos < limit) value = value + x;
            } else {
                const bool better = MODE == STAT_MIN ? x < value : x > value;
                if (pos < limit && (pos == 0 || better)) { value = x; found = pos; }
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
    // The next level of the tree in the same launch: the piece's 256 tile results are 256 / RTS whole tiles of the
    // next level; one thread each reduces them front to back out of LDS and only those results are written.
    level_val[threadIdx.x] = value;
    if (INDEXED && limit > 0) {
        const int64_t at = my_first + found;                          // position in this level's input
        level_idx[threadIdx.x] = idx_in ? idx_in[at] : (int)at;       // ... mapped back to the original data
    }
    __syncthreads();
    if (threadIdx.x < NEXT) {
        const int64_t results = (n + RTS - 1) / RTS;                  // tile results of this level in the whole grid
        const int64_t first = piece * 256 + (int64_t)threadIdx.x * RTS;
        if (first < results) {
            const int count = results - first < RTS ? (int)(results - first) : RTS;
            T v = T(0);
            int at = 0;
            auto take = [&](T x, int i) {
                if (!INDEXED) v = v + x;
                else {
                    const bool better = MODE == STAT_MIN ? x < v : x > v;
                    if (i == 0 || better) { v = x; at = i; }
                }
            };
            if (count == RTS) {
                // a whole tile: sixteen values per trip through 16-byte LDS reads that are all requested before the
                // first is used (one value per trip would wait out an LDS latency RTS times, at the end of every block)
                constexpr int STEP = 16;
                typedef T Vec __attribute__((ext_vector_type(VEC)));
                for (int i0 = 0; i0 < RTS; i0 += STEP) {
                    Vec q[STEP / VEC];
#pragma unroll
                    for (int k = 0; k < STEP / VEC; k++) q[k] = *(const Vec*)(&level_val[threadIdx.x * RTS + i0 + k * VEC]);
#pragma unroll
                    for (int k = 0; k < STEP / VEC; k++)
#pragma unroll
                        for (int e = 0; e < VEC; e++) take(q[k][e], i0 + k * VEC + e);
                }
            } else {
                for (int i = 0; i < count; i++) take(level_val[threadIdx.x * RTS + i], i);
            }
            out[piece * NEXT + threadIdx.x] = v;
            if (INDEXED) idx_out[piece * NEXT + threadIdx.x] = level_idx[threadIdx.x * RTS + at];
        }
    }
    if (piece_i + 1 < pieces) __syncthreads();       // the next piece overwrites level_val / level_idx
    }
}

// The last levels in one launch: once at most 256 tiles are left, one block finishes the tree.  Thread t reduces
// tile t straight from memory (a whole tile is requested at once, then combined front to back), the tile results
// go to LDS, and the following levels -- at most 256 values, then at most 4 -- are reduced there the same way.
template <typename T, int RTS, int MODE>
__global__ __launch_bounds__(256) void tail_reduce_kernel(const T* __restrict__ in, const T* __restrict__ in2,
                                                          const int* __restrict__ idx_in, int m,
                                                          T* __restrict__ out, int* __restrict__ idx_out) {
    constexpr int VEC = 16 / sizeof(T);
    typedef T Vec __attribute__((ext_vector_type(VEC), aligned(sizeof(T))));      // partial results start at any element
    constexpr bool INDEXED = MODE == STAT_MIN || MODE == STAT_MAX;
    __shared__ T vals[2][256];
    __shared__ int idxs[2][256];
    const int t = threadIdx.x;
    int count = (m + RTS - 1) / RTS;                 // <= 256, checked by the host
    auto combine = [&](T& value, int& found, T x, int pos) {
        if (MODE == STAT_SUM || MODE == STAT_DOT) value = value + x;
        else {
            const bool better = MODE == STAT_MIN ? x < value : x > value;
            if (pos == 0 || better) { value = x; found = pos; }
        }
    };
    if (t < count) {
        const int first = t * RTS;
        const int limit = m - first < RTS ? m - first : RTS;
        T value = T(0);
        int found = 0;
        if (limit == RTS) {
            Vec v[RTS / VEC], w[RTS / VEC];
#pragma unroll
            for (int k = 0; k < RTS / VEC; k++) {
                v[k] = ((const Vec*)(in + first))[k];
                if (MODE == STAT_DOT) w[k] = ((const Vec*)(in2 + first))[k];
            }
#pragma unroll
            for (int k = 0; k < RTS / VEC; k++)
#pragma unroll
                for (int e = 0; e < VEC; e++) combine(value, found, MODE == STAT_DOT ? v[k][e] * w[k][e] : v[k][e], k * VEC + e);
        } else {
            for (int i = 0; i < limit; i++) combine(value, found, MODE == STAT_DOT ? in[first + i] * in2[first + i] : in[first + i], i);
        }
        vals[0][t] = value;
        if (INDEXED) idxs[0][t] = idx_in ? idx_in[first + found] : first + found;
    }
    __syncthreads();
    int cur = 0;
    while (count > 1) {
        const int next = (count + RTS - 1) / RTS;
        if (t < next) {
            const int first = t * RTS;
            const int limit = count - first < RTS ? count - first : RTS;
            T value = T(0);
            int found = 0;
            for (int i = 0; i < limit; i++) {
                const T x = vals[cur][first + i];
                if (MODE == STAT_SUM || MODE == STAT_DOT) value = value + x;
                else {
                    const bool better = MODE == STAT_MIN ? x < value : x > value;
                    if (i == 0 || better) { value = x; found = i; }
                }
            }
            vals[cur ^ 1][t] = value;
            if (INDEXED) idxs[cur ^ 1][t] = idxs[cur][first + found];
        }
        __syncthreads();
        cur ^= 1;
        count = next;
    }
    if (t == 0) {
        out[0] = vals[cur][0];
        if (INDEXED) idx_out[0] = idxs[cur][0];
    }
}

// Partial results reduce_levels keeps for n elements: what every launch but the last writes (a launch covers two
// levels of the tree) plus one slot for the last; values first, then, from the next 16-byte boundary, their indices.
template <int RTS>
static int64_t partial_slots(int64_t n) {
    int64_t total = 1, m = n;
    while ((m + RTS - 1) / RTS > 256) { m = ((m + RTS - 1) / RTS + RTS - 1) / RTS; total += m; }
    return total;
}
template <typename T, int RTS>
static uint64_t partials_bytes(int64_t n) {
    const uint64_t total = (uint64_t)partial_slots<RTS>(n);
    return ((total * sizeof(T) + 15) & ~(uint64_t)15) + total * sizeof(int);
}

// `scratch` (of at least partials_bytes<T, RTS>(n) bytes) holds the partial results; nullptr takes the device
// workspace, which is grown (allocated) on demand.
template <typename T, int RTS, int MODE>
static int reduce_levels(Device* dev, const T* in, const T* in2, int64_t n, T* out_value, int* out_index,
                         void* scratch = nullptr) {
    constexpr bool indexed = MODE == STAT_MIN || MODE == STAT_MAX;
    if (MODE == STAT_SUM && n == 1) {               // CPUSum returns a single element as it is (keeps a -0)
        NK_HIP(hipMemcpyAsync(out_value, in, sizeof(T), hipMemcpyDeviceToDevice, dev->stream));
        return NK_OK;
    }
    const int64_t total = partial_slots<RTS>(n);
    void* ws = scratch;
    if (!ws) if (int e = workspace(dev, partials_bytes<T, RTS>(n), &ws)) return e;
    T* vals = (T*)ws;
    int* idxs = (int*)((char*)ws + (((uint64_t)total * sizeof(T) + 15) & ~(uint64_t)15));
    const T* cur = in;
    const T* cur2 = in2;
    const int* cur_idx = nullptr;
    int64_t m = n, used = 0;
    int level = 0;
    do {
        const int64_t tiles = (m + RTS - 1) / RTS;
        if (tiles <= 256) {                         // one block finishes the tree
            T* dst = out_value ? out_value : vals + used;
            int* dst_idx = !indexed ? nullptr : (out_index ? out_index : idxs + used);
            if (MODE == STAT_DOT && level > 0)
                hipLaunchKernelGGL((tail_reduce_kernel<T, RTS, STAT_SUM>), dim3(1), dim3(256), 0, dev->stream, cur, cur, cur_idx, (int)m, dst, dst_idx);
            else
                hipLaunchKernelGGL((tail_reduce_kernel<T, RTS, MODE>), dim3(1), dim3(256), 0, dev->stream, cur, cur2, cur_idx, (int)m, dst, dst_idx);
            break;
        }
        T* dst = vals + used;
        int* dst_idx = indexed ? idxs + used : nullptr;
        // pieces of 256 tiles; a block walks several consecutive ones so that about two blocks per compute unit exist
        // (sum of 2^26 floats: one block per unit 60.6 us, two 43.6, four 45.8, eight 44.2, one piece per block 45.1)
        const int64_t piece_count = (tiles + 255) / 256;
        const int64_t two_per_cu = 2 * (int64_t)dev->props.multiProcessorCount;
        const int pieces = (int)(piece_count > two_per_cu ? (piece_count + two_per_cu - 1) / two_per_cu : 1);
        const unsigned blocks = (unsigned)((piece_count + pieces - 1) / pieces);
        if (MODE == STAT_DOT && level > 0)
            hipLaunchKernelGGL((tile_reduce_kernel<T, RTS, STAT_SUM>), dim3(blocks), dim3(256), 0, dev->stream, cur, cur, cur_idx, m, dst, dst_idx, pieces);
        else
            hipLaunchKernelGGL((tile_reduce_kernel<T, RTS, MODE>), dim3(blocks), dim3(256), 0, dev->stream, cur, cur2, cur_idx, m, dst, dst_idx, pieces);
        cur = dst; cur2 = dst; cur_idx = dst_idx;
        const int64_t written = (tiles + RTS - 1) / RTS;           // the launch covers two levels of the tree
        used += written;
        m = written;
        level += 2;
    } while (m > 1);
    NK_HIP(hipGetLastError());
    return NK_OK;
}

static int check_vector(Device* dev, const char* what, int dtype, nk_buf buf, int64_t n) {
    NK_REQUIRE(dtype == NK_F32 || dtype == NK_F64, "%s: unknown dtype %d", what, dtype);
    NK_REQUIRE(n >= 1 && n < ((int64_t)1 << 31), "%s: n = %lld outside [1, 2^31)", what, (long long)n);
    NK_REQUIRE(buf % 16 == 0, "%s: the data must start on a 16-byte boundary", what);
    return check_range(dev, what, buf, 0, (uint64_t)n * dtype_bytes(dtype));
}

}  // namespace nk

using namespace nk;

extern "C" int nk_sum(nk_dev h, int dtype, nk_buf in, int64_t n, nk_buf out) {
    NK_DEVICE(dev, h);
    if (int e = check_vector(dev, "nk_sum(in)", dtype, in, n)) return e;
    if (int e = check_range(dev, "nk_sum(out)", out, 0, dtype_bytes(dtype))) return e;
    set_path("tile_tree_128");
    return dtype == NK_F32 ? reduce_levels<float, 128, STAT_SUM>(dev, (const float*)in, nullptr, n, (float*)out, nullptr)
                           : reduce_levels<double, 128, STAT_SUM>(dev, (const double*)in, nullptr, n, (double*)out, nullptr);
}

// nk_sum for callers that cannot allocate: the partial results live in a file-scope device array instead of the
// device workspace.  The array's name is a host-side stand-in, not a device address; the address is asked for once
// per opened device (with that device current) and only that pointer is handed to the kernels.
constexpr uint64_t SUM_STATIC_BYTES = 1u << 20;
static __device__ __align__(256) unsigned char scratch[SUM_STATIC_BYTES];

int nk::stats_static_init(Device* dev) {
    void* ptr = nullptr;
    NK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    dev->sum_static_scratch = ptr;
    return NK_OK;
}

extern "C" int nk_sum_static(nk_dev h, int dtype, nk_buf in, int64_t n, nk_buf out) {
    NK_DEVICE(dev, h);
    NK_REQUIRE(n <= NK_SUM_STATIC_MAX_N, "nk_sum_static: n = %lld exceeds the maximum of %lld elements this entry point "
               "holds partial results for; use nk_sum", (long long)n, (long long)NK_SUM_STATIC_MAX_N);
    if (int e = check_vector(dev, "nk_sum_static(in)", dtype, in, n)) return e;
    if (int e = check_range(dev, "nk_sum_static(out)", out, 0, dtype_bytes(dtype))) return e;
    const uint64_t need = dtype == NK_F32 ? partials_bytes<float, 128>(n) : partials_bytes<double, 128>(n);
    NK_REQUIRE(need <= SUM_STATIC_BYTES, "nk_sum_static: %llu bytes of partial results exceed the static scratch",
               (unsigned long long)need);
    NK_REQUIRE(dev->sum_static_scratch != nullptr, "nk_sum_static: the static scratch of this device was not resolved");
    set_path("tile_tree_128_static");
    // every partial slot a launch reads was written by the launch before it, so nothing has to start at zero
    return dtype == NK_F32
        ? reduce_levels<float, 128, STAT_SUM>(dev, (const float*)in, nullptr, n, (float*)out, nullptr, dev->sum_static_scratch)
        : reduce_levels<double, 128, STAT_SUM>(dev, (const double*)in, nullptr, n, (double*)out, nullptr, dev->sum_static_scratch);
}

extern "C" int nk_reduce_index(nk_dev h, int kind, int dtype, nk_buf in, int64_t n, nk_buf out_index) {
    NK_DEVICE(dev, h);
    NK_REQUIRE(kind == NK_REDUCE_MIN || kind == NK_REDUCE_MAX, "nk_reduce_index: unknown kind %d", kind);
    if (int e = check_vector(dev, "nk_reduce_index(in)", dtype, in, n)) return e;
    if (int e = check_range(dev, "nk_reduce_index(out)", out_index, 0, sizeof(int))) return e;
    set_path("tile_tree_64");
    if (dtype == NK_F32)
        return kind == NK_REDUCE_MIN ? reduce_levels<float, 64, STAT_MIN>(dev, (const float*)in, nullptr, n, nullptr, (int*)out_index)
                                     : reduce_levels<float, 64, STAT_MAX>(dev, (const float*)in, nullptr, n, nullptr, (int*)out_index);
    return kind == NK_REDUCE_MIN ? reduce_levels<double, 64, STAT_MIN>(dev, (const double*)in, nullptr, n, nullptr, (int*)out_index)
                                 : reduce_levels<double, 64, STAT_MAX>(dev, (const double*)in, nullptr, n, nullptr, (int*)out_index);
}

extern "C" int nk_dot(nk_dev h, int dtype, nk_buf a, nk_buf b, int64_t n, nk_buf out) {
    NK_DEVICE(dev, h);
    if (int e = check_vector(dev, "nk_dot(a)", dtype, a, n)) return e;
    if (int e = check_vector(dev, "nk_dot(b)", dtype, b, n)) return e;
    if (int e = check_range(dev, "nk_dot(out)", out, 0, dtype_bytes(dtype))) return e;
    set_path("tile_tree_128");
    return dtype == NK_F32 ? reduce_levels<float, 128, STAT_DOT>(dev, (const float*)a, (const float*)b, n, (float*)out, nullptr)
                           : reduce_levels<double, 128, STAT_DOT>(dev, (const double*)a, (const double*)b, n, (double*)out, nullptr);
}
