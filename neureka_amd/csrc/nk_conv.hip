// nk_convolution: the reference's 'x' operator (nd valid cross-correlation) and its gradient.
//
// Semantics (J/backend/main/implementations/convolution/AbstractCPUConvolution.java:245-408):
//   forward  drain[o] = sum_j src1[b1 + j] * src2[b2 + j],  j over prod_k [0, min(s1[k], s2[k])),
//            b1[k] = s1[k] >= s2[k] ? o[k] : 0,  b2[k] = s1[k] <= s2[k] ? o[k] : 0, axis 0 fastest
//   gradient drain[o] = sum_e [0 <= i1 < s1] src1[i1] * src2[e],  e over all of src2, axis 0 fastest,
//            i1[k] = s0[k] > s1[k] ? o[k] - e[k] : o[k] + e[k]
//
// Kernels
//   literal        any rank / layout / view: one thread per drain element, the sum in the reference's
//                  order with rounded products, bit-identical to the CPU device.  The gradient only
//                  visits the e-range that can pass the bounds test (skipped terms add +0).
//   split          the same terms where one thread per drain element would leave the machine idle (long sums into few
//                  elements): a wavefront or a block per element, in segments if need be; re-ordered sum.
//   chan_fwd/dx/dk rank 3, dense row-major f32, full reduction over axis 0 (channels), square taps of extent
//                  2, 3, 4, 5 or 7: [C,H,W] x [C,k,k] -> [1,H-k+1,W-k+1] and its two gradients, register
//                  sliding-window kernels (see below); sums are re-ordered, results agree with the reference
//                  norm-wise (1e-5 * sum |a||b| per output).
#include "nk_internal.h"
#include <type_traits>
#include <cstdlib>

namespace nk {

struct ConvArgs {
    int rank;
    unsigned n;
    Cfg c0, c1, c2;
};

template <typename T, int RANK>
__global__ __launch_bounds__(256) void conv_fwd_literal(ConvArgs A, T* __restrict__ drn, const T* __restrict__ s1,
                                                        const T* __restrict__ s2) {
    const unsigned step = gridDim.x * blockDim.x;
    const int rank = RANK ? RANK : A.rank;          // RANK = 0: any rank up to NK_MAX_RANK
    constexpr int NR = RANK ? RANK : NK_MAX_RANK;
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < A.n; i += step) {
        int o[NR], b1[NR], b2[NR], j[NR], m[NR];
        nd_of_flat(A.c0, rank, (int)i, o);
        for (int k = 0; k < rank; k++) {
            const int e1 = A.c1.shape[k], e2 = A.c2.shape[k];
            b1[k] = e1 >= e2 ? o[k] : 0;
            b2[k] = e1 <= e2 ? o[k] : 0;
            m[k] = e1 < e2 ? e1 : e2;
            j[k] = 0;
        }
        T value = T(0);
        bool running = true;
        while (running) {
            int i1[NR], i2[NR];
            for (int k = 0; k < rank; k++) { i1[k] = b1[k] + j[k]; i2[k] = b2[k] + j[k]; }
            T prod = s1[phys_of_nd(A.c1, rank, i1)] * s2[phys_of_nd(A.c2, rank, i2)];
            value = value + prod;
            int k = 0;
            for (; k < rank; k++) {
                if (++j[k] < m[k]) break;
                j[k] = 0;
            }
            running = k < rank;
        }
        drn[phys_of_nd(A.c0, rank, o)] = value;
    }
}

template <typename T, int RANK>
__global__ __launch_bounds__(256) void conv_bwd_literal(ConvArgs A, T* __restrict__ drn, const T* __restrict__ s1,
                                                        const T* __restrict__ s2) {
    const unsigned step = gridDim.x * blockDim.x;
    const int rank = RANK ? RANK : A.rank;          // RANK = 0: any rank up to NK_MAX_RANK
    constexpr int NR = RANK ? RANK : NK_MAX_RANK;
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < A.n; i += step) {
        int o[NR], lo[NR], hi[NR], e[NR];
        nd_of_flat(A.c0, rank, (int)i, o);
        bool empty = false;
        for (int k = 0; k < rank; k++) {
            const int e0 = A.c0.shape[k], e1 = A.c1.shape[k], e2 = A.c2.shape[k];
            if (e0 > e1) {            // i1 = o - e in [0, e1)
                lo[k] = o[k] - e1 + 1; if (lo[k] < 0) lo[k] = 0;
                hi[k] = o[k] + 1;      if (hi[k] > e2) hi[k] = e2;
            } else {                  // i1 = o + e in [0, e1)
                lo[k] = 0;
                hi[k] = e1 - o[k];     if (hi[k] > e2) hi[k] = e2;
            }
            if (hi[k] <= lo[k]) empty = true;
            e[k] = lo[k];
        }
        T value = T(0);
        bool running = !empty;
        while (running) {
            int i1[NR];
            for (int k = 0; k < rank; k++) i1[k] = A.c0.shape[k] > A.c1.shape[k] ? o[k] - e[k] : o[k] + e[k];
            T prod = s1[phys_of_nd(A.c1, rank, i1)] * s2[phys_of_nd(A.c2, rank, e)];
            value = value + prod;
            int k = 0;
            for (; k < rank; k++) {
                if (++e[k] < hi[k]) break;
                e[k] = lo[k];
            }
            running = k < rank;
        }
        drn[phys_of_nd(A.c0, rank, o)] = value;
    }
}

// Long sums into few drain elements (a tap gradient, a full reduction over channels in f64, ...): with one
// thread per drain element the machine would idle behind a handful of very long serial sums.  Here a block
// owns a drain element: its 256 threads take every 256th term -- enumerated with the last axis fastest, the
// order memory runs in for row-major operands -- and their partial sums meet in a fixed LDS tree.  Each thread
// steps its nd term index by 256 with a mixed-radix add (no division inside the loop).  Same terms as the
// literal kernels, another order: results agree with the reference norm-wise, not bit for bit.
// GS lanes per drain element: 256 (a block) or 64 (a wavefront, four elements per block) for sums that are only a
// few hundred terms long.  SEG: the terms of an element are cut into gridDim.y segments whose partial sums go to
// `partial` and are added in order by conv_split_finish (very few elements, very long sums: a tap gradient).
struct SplitArgs {
    unsigned per_xcd;        // element groups per XCD (the grid's x extent is 8 * per_xcd)
    unsigned seg_terms;      // SEG: terms per segment
};

template <typename T, bool BWD, int RANK, int GS, bool SEG>
__global__ __launch_bounds__(256) void conv_split(ConvArgs A, SplitArgs S, T* __restrict__ drn, T* __restrict__ partial,
                                                  const T* __restrict__ s1, const T* __restrict__ s2) {
    constexpr int EPB = 256 / GS;                   // drain elements per block
    __shared__ T part[256];
    const int tid = threadIdx.x;
    const unsigned lane = (unsigned)tid % GS, sub = (unsigned)tid / GS;
    const int rank = RANK ? RANK : A.rank;          // RANK = 0: any rank up to NK_MAX_RANK
    constexpr int NR = RANK ? RANK : NK_MAX_RANK;
    // consecutive block ids go round-robin to the 8 XCDs: give every XCD one contiguous eighth of the drain, so that
    // neighbouring drain elements, whose terms overlap, share that XCD's L2
    const unsigned group = (blockIdx.x & 7u) * S.per_xcd + (blockIdx.x >> 3);
    const unsigned i = group * EPB + sub;
    const bool live = i < A.n;
    int o[NR], lo[NR], ext[NR], b1[NR], j[NR], d[NR];
    nd_of_flat(A.c0, rank, (int)(live ? i : 0), o);
    unsigned terms = 1;
    for (int k = 0; k < rank; k++) {
        const int e0 = A.c0.shape[k], e1 = A.c1.shape[k], e2 = A.c2.shape[k];
        if (!BWD) {
            b1[k] = e1 >= e2 ? o[k] : 0;
            lo[k] = e1 <= e2 ? o[k] : 0;                 // start in src2
            ext[k] = e1 < e2 ? e1 : e2;
        } else {
            int l, h;
            if (e0 > e1) { l = o[k] - e1 + 1; if (l < 0) l = 0; h = o[k] + 1; if (h > e2) h = e2; }
            else         { l = 0; h = e1 - o[k]; if (h > e2) h = e2; }
            lo[k] = l;
            ext[k] = h > l ? h - l : 0;
            b1[k] = 0;
        }
        terms *= (unsigned)ext[k];
    }
    unsigned first = 0, end = terms;
    if (SEG) {
        first = blockIdx.y * S.seg_terms;
        end = first + S.seg_terms < terms ? first + S.seg_terms : terms;
    }
    T value = T(0);
    if (live && first < end) {
        unsigned r = first + lane, q = (unsigned)GS;
        for (int k = rank - 1; k >= 0; k--) {
            j[k] = (int)(r % (unsigned)ext[k]); r /= (unsigned)ext[k];
            d[k] = (int)(q % (unsigned)ext[k]); q /= (unsigned)ext[k];
        }
#pragma unroll 4
        for (unsigned t = first + lane; t < end; t += (unsigned)GS) {
            int i1[NR], i2[NR];
            for (int k = 0; k < rank; k++) {
                i2[k] = lo[k] + j[k];
                if (!BWD) i1[k] = b1[k] + j[k];
                else      i1[k] = A.c0.shape[k] > A.c1.shape[k] ? o[k] - i2[k] : o[k] + i2[k];
            }
            const T prod = s1[phys_of_nd(A.c1, rank, i1)] * s2[phys_of_nd(A.c2, rank, i2)];
            value = value + prod;
            int carry = 0;
            for (int k = rank - 1; k >= 0; k--) {
                j[k] += d[k] + carry;
                carry = j[k] >= ext[k];
                if (carry) j[k] -= ext[k];
            }
        }
    }
    part[tid] = value;
    __syncthreads();
    for (int w = GS / 2; w > 0; w >>= 1) {
        if ((int)lane < w) part[tid] = part[tid] + part[tid + w];
        __syncthreads();
    }
    if (lane == 0 && live) {
        if (SEG) partial[(int64_t)blockIdx.y * A.n + i] = part[tid];
        else drn[phys_of_nd(A.c0, rank, o)] = part[tid];
    }
}

template <typename T>
__global__ __launch_bounds__(256) void conv_split_finish(Cfg c0, int rank, unsigned n, int segments, const T* __restrict__ partial, T* __restrict__ drn) {
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    T s = T(0);
    for (int k = 0; k < segments; k++) s = s + partial[(int64_t)k * n + i];
    drn[phys_of_flat(c0, rank, (int)i)] = s;
}

// ------------------------------------------------------------------------------------------------
// Channel convolution, dense row-major f32: big [C,H,W], taps [C,KH,KW], out/err [1,OH,OW], OH = H-KH+1.
//
// All three kernels give a lane CX = 4 adjacent columns and a strip of rows and keep the window they work
// on in registers: the 4 + KW - 1 values a row contributes are reused across the KW horizontal and the KH
// vertical shifts without touching memory again.  Row bases are wave-uniform (scalar unit); a lane adds a
// 32-bit byte offset computed once, so the vector unit spends its issue slots on multiply-adds instead of
// 64-bit address arithmetic.  Dead lanes and rows past the end read clamped, valid addresses and their
// results are dropped, which keeps every load unconditional.  The per-channel taps are wave-uniform and come
// in through scalar loads.  Extents of the taps are template parameters so every loop is unrolled and every
// accumulator lives in a register.  Work is split over channel groups (or strips) until there are enough
// wavefronts to fill the machine; partial results go to a device-owned scratch buffer and a second pass
// adds them in a fixed order (deterministic, no atomics).
struct ChanArgs {
    int C, H, W, OH, OW;
    int cg;              // channels per group (grid z)
    int col_blocks;      // 256-column blocks across the lane axis
    int err_plane;       // gradients: elements between the error planes of two channels (0: one plane for all)
    int tap_plane;       // gradients: elements between the taps of two channels (0: one set for all)
};

template <typename T>
__global__ __launch_bounds__(256) void conv_partial_reduce(int parts, int n, const T* __restrict__ partial, T* __restrict__ out) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    T s = T(0);
    int k = 0;
    for (; k + 8 <= parts; k += 8) {              // eight independent loads in flight, added in a fixed order
        T v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = partial[(int64_t)(k + u) * n + i];
#pragma unroll
        for (int u = 0; u < 8; u++) s = s + v[u];
    }
    for (; k < parts; k++) s = s + partial[(int64_t)k * n + i];
    out[i] = s;
}

// few outputs, many partials (the tap gradient): one wavefront per output, lanes stride over the partials
template <typename T>
__global__ __launch_bounds__(256) void conv_partial_reduce_wide(int parts, int n, const T* __restrict__ partial, T* __restrict__ out) {
    const int i = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (i >= n) return;
    T s = T(0);
    for (int k = lane; k < parts; k += 64) s = s + partial[(int64_t)k * n + i];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) s += __shfl_down(s, off, 64);
    if (lane == 0) out[i] = s;
}

constexpr int CX = 4;                       // columns per lane
typedef float f32x4u __attribute__((ext_vector_type(4), aligned(4)));
typedef double f64x2u __attribute__((ext_vector_type(2), aligned(8)));
typedef int i32x2 __attribute__((ext_vector_type(2)));

// one fused multiply-add in the operand's own precision (the bare builtin is the double one)
__device__ __forceinline__ float fused_mad(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double fused_mad(double a, double b, double c) { return __builtin_fma(a, b, c); }

// Buffer addressing: a wave-uniform descriptor (base, extent in bytes) in scalar registers, a scalar byte
// offset for the row and one 32-bit per-lane byte offset -- no 64-bit vector arithmetic per access.  The
// extent must stay below 2^32 bytes (checked on the host).
typedef __amdgpu_buffer_rsrc_t BufRsrc;
__device__ __forceinline__ BufRsrc buffer_of(const void* base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, bytes, 0x00020000);      // raw buffer, 32-bit data format
}
__device__ __forceinline__ float buffer_load(BufRsrc r, unsigned lane_off, unsigned row_off) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, lane_off, row_off, 0));
}
__device__ __forceinline__ f32x4u buffer_load4(BufRsrc r, unsigned lane_off, unsigned row_off) {
    return __builtin_bit_cast(f32x4u, __builtin_amdgcn_raw_buffer_load_b128(r, lane_off, row_off, 0));
}

__device__ __forceinline__ int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

// Rows are addressed through one buffer descriptor per row (base = first element of the row, extent = the row):
// the hardware range check then returns 0 for every dword left or right of the row (negative lane offsets wrap to
// huge unsigned ones) and, with an extent of 0, for a whole row that does not exist.  No clamp, no mask.
template <typename T>
__device__ __forceinline__ BufRsrc row_of(const T* base, int64_t row, int width, bool exists) {
    return buffer_of(base + (exists ? row * width : 0), exists ? (unsigned)width * (unsigned)sizeof(T) : 0u);
}

// the CX columns col .. col+CX-1 of a row (col is a multiple of CX and may lie left or right of the row): one
// 16-byte load in f32, two in f64
__device__ __forceinline__ void load_cols(BufRsrc row, int col, float* dst) {
    const f32x4u q = buffer_load4(row, (unsigned)col * 4u, 0);
#pragma unroll
    for (int e = 0; e < CX; e++) dst[e] = q[e];
}
__device__ __forceinline__ void load_cols(BufRsrc row, int col, double* dst) {
    const unsigned off = (unsigned)col * 8u;
    const f64x2u lo = __builtin_bit_cast(f64x2u, __builtin_amdgcn_raw_buffer_load_b128(row, off, 0, 0));
    const f64x2u hi = __builtin_bit_cast(f64x2u, __builtin_amdgcn_raw_buffer_load_b128(row, off + 16u, 0, 0));
    dst[0] = lo[0]; dst[1] = lo[1]; dst[2] = hi[0]; dst[3] = hi[1];
}
// CX adjacent results that nothing reads again soon
__device__ __forceinline__ void store_cols(float* dst, const float* v) {
    f32x4u o; o[0] = v[0]; o[1] = v[1]; o[2] = v[2]; o[3] = v[3];
    __builtin_nontemporal_store(o, (f32x4u*)dst);
}
__device__ __forceinline__ void store_cols(double* dst, const double* v) {
    f64x2u lo, hi; lo[0] = v[0]; lo[1] = v[1]; hi[0] = v[2]; hi[1] = v[3];
    __builtin_nontemporal_store(lo, (f64x2u*)dst);
    __builtin_nontemporal_store(hi, (f64x2u*)dst + 1);
}

// A lane holds CX adjacent columns; the KW - 1 further columns its window needs are the first (forward) or last
// (gradients) registers of its neighbours.  They arrive through wavefront shifts of the registers instead of
// through more loads: one load of CX columns per lane and row is all the memory traffic a window costs.  Only the
// lane at the end (start) of the wavefront, which has no neighbour, loads its extra columns itself; the shift
// leaves that lane's registers as they are.  A double moves as its two halves.
__device__ __forceinline__ float from_next_lane(float keep, float v) {     // lane i <- lane i + 1, lane 63 keeps `keep`
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, keep), __builtin_bit_cast(int, v), 0x130, 0xf, 0xf, false));
}
__device__ __forceinline__ float from_prev_lane(float keep, float v) {     // lane i <- lane i - 1, lane 0 keeps `keep`
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, keep), __builtin_bit_cast(int, v), 0x138, 0xf, 0xf, false));
}
__device__ __forceinline__ double from_next_lane(double keep, double v) {
    const i32x2 k = __builtin_bit_cast(i32x2, keep), s = __builtin_bit_cast(i32x2, v);
    i32x2 r;
    r[0] = __builtin_amdgcn_update_dpp(k[0], s[0], 0x130, 0xf, 0xf, false);
    r[1] = __builtin_amdgcn_update_dpp(k[1], s[1], 0x130, 0xf, 0xf, false);
    return __builtin_bit_cast(double, r);
}
__device__ __forceinline__ double from_prev_lane(double keep, double v) {
    const i32x2 k = __builtin_bit_cast(i32x2, keep), s = __builtin_bit_cast(i32x2, v);
    i32x2 r;
    r[0] = __builtin_amdgcn_update_dpp(k[0], s[0], 0x138, 0xf, 0xf, false);
    r[1] = __builtin_amdgcn_update_dpp(k[1], s[1], 0x138, 0xf, 0xf, false);
    return __builtin_bit_cast(double, r);
}
// Sum over the 64 lanes of a wavefront, delivered in lane 63, with data-parallel-primitive adds instead of LDS
// permutes: four shifted adds inside each row of 16 lanes (lane 15 of a row then holds the row's sum), then lane 15
// of rows 0 and 2 is added into rows 1 and 3, then lane 31 into rows 2 and 3.  Lanes a step does not reach, or
// whose source lies outside the row, add zero.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_or_zero(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false));
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_or_zero(double v) {
    const i32x2 s = __builtin_bit_cast(i32x2, v);
    i32x2 r;
    r[0] = __builtin_amdgcn_update_dpp(0, s[0], CTRL, ROW_MASK, 0xf, false);
    r[1] = __builtin_amdgcn_update_dpp(0, s[1], CTRL, ROW_MASK, 0xf, false);
    return __builtin_bit_cast(double, r);
}
template <typename T>
__device__ __forceinline__ T wave_sum_in_lane63(T v) {
    v += dpp_or_zero<0x111, 0xf>(v);        // row_shr:1
    v += dpp_or_zero<0x112, 0xf>(v);        // row_shr:2
    v += dpp_or_zero<0x114, 0xf>(v);        // row_shr:4
    v += dpp_or_zero<0x118, 0xf>(v);        // row_shr:8
    v += dpp_or_zero<0x142, 0xa>(v);        // row_bcast:15 into rows 1 and 3
    v += dpp_or_zero<0x143, 0xc>(v);        // row_bcast:31 into rows 2 and 3
    return v;
}
constexpr int WAVE_COLS = 64 * CX;          // columns per wavefront

// CX adjacent results through ordinary 16-byte stores
__device__ __forceinline__ void write_cols(float* dst, const float* v) {
    f32x4u o; o[0] = v[0]; o[1] = v[1]; o[2] = v[2]; o[3] = v[3];
    *(f32x4u*)dst = o;
}
__device__ __forceinline__ void write_cols(double* dst, const double* v) {
    f64x2u lo, hi; lo[0] = v[0]; lo[1] = v[1]; hi[0] = v[2]; hi[1] = v[3];
    *(f64x2u*)dst = lo;
    *((f64x2u*)dst + 1) = hi;
}

// The KW - 1 columns a lane's window needs beyond its own CX come from its neighbour's registers; only the lane at
// the end of the wavefront has no neighbour and loads them.  That load carries no branch: every other lane asks for
// a column far outside the row, which the range check of the row's descriptor answers with 0 without a memory
// access.  A branch around it (`if (lane == 63)`) makes the compiler close the divergent block with a wait for the
// load -- one exposed round trip per window row, twelve in a row for a 5 x 5 tap gradient.  Without it the edge
// loads leave with the row's other loads and one wait covers them all.
constexpr int FAR_COL = 0x3FFFFFF8;         // times 4 or 8 bytes, and the next 32 bytes, still beyond every row (a plane, so a row, stays below 2 GiB: checked on the host)

// window[0 .. CX-1] holds (or will hold) the lane's own columns x .. x+CX-1 of `row`; requests, in the last lane,
// the columns to the right of them into window[CX .. CX+EXTRA-1] (0 in every other lane)
template <int EXTRA, typename T>
__device__ __forceinline__ void request_right(T (&window)[CX + EXTRA], BufRsrc row, int x, int lane) {
    static_assert(EXTRA <= 2 * CX, "at most two further pieces of CX columns");
    T a[CX];
    load_cols(row, lane == 63 ? x + CX : FAR_COL, a);
#pragma unroll
    for (int e = 0; e < CX && e < EXTRA; e++) window[CX + e] = a[e];
    if (EXTRA > CX) {
        T b[CX];
        load_cols(row, lane == 63 ? x + 2 * CX : FAR_COL, b);
#pragma unroll
        for (int e = CX; e < EXTRA; e++) window[CX + e] = b[e - CX];
    }
}
// after request_right and the loads of the own columns: every lane but the last takes its neighbour's columns
template <int EXTRA, typename T>
__device__ __forceinline__ void shift_in_right(T (&window)[CX + EXTRA]) {
#pragma unroll
    for (int e = CX; e < CX + EXTRA; e++) window[e] = from_next_lane(window[e], window[e - CX]);
}

// window[EXTRA .. EXTRA+CX-1] holds (or will hold) the lane's own columns x .. x+CX-1 of `row`; requests, in the
// first lane, the columns x-EXTRA .. x-1 to the left of them into window[0 .. EXTRA-1] (columns left of the row
// start read as zero, as does every other lane)
template <int EXTRA, typename T>
__device__ __forceinline__ void request_left(T (&window)[CX + EXTRA], BufRsrc row, int x, int lane) {
    static_assert(EXTRA <= 2 * CX, "at most two further pieces of CX columns");
    T a[CX];
    load_cols(row, lane == 0 ? x - CX : FAR_COL, a);                       // columns x-4 .. x-1
#pragma unroll
    for (int e = 0; e < CX; e++) if (EXTRA - CX + e >= 0) window[EXTRA - CX + e] = a[e];
    if (EXTRA > CX) {
        T b[CX];
        load_cols(row, lane == 0 ? x - 2 * CX : FAR_COL, b);               // columns x-8 .. x-5
#pragma unroll
        for (int e = 0; e < CX; e++) if (EXTRA - 2 * CX + e >= 0) window[EXTRA - 2 * CX + e] = b[e];
    }
}
template <int EXTRA, typename T>
__device__ __forceinline__ void shift_in_left(T (&window)[CX + EXTRA]) {
#pragma unroll
    for (int i = EXTRA - 1; i >= 0; i--) window[i] = from_prev_lane(window[i], window[i + CX]);
}

// forward: partial[z][y][x] = sum_{c in group z} sum_ky sum_kx in[c][y+ky][x+kx] * w[c][ky][kx]
// block -> (column block, strip of R output rows, channel group); its NW wavefronts take every NW-th channel of
// the group and are summed through LDS in a fixed order before the block writes its (partial) plane.  With
// NW = 16 and one group the block reduces all channels itself and no second pass is needed.
template <typename T, int KH, int KW, int R, int NW>
__global__ __launch_bounds__(NW * 64) void conv_chan_fwd(ChanArgs g, const T* __restrict__ in, const T* __restrict__ w, T* __restrict__ partial) {
    constexpr int COLS = WAVE_COLS;
    __shared__ T red[NW][R][64 * CX];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int x = blockIdx.x * COLS + lane * CX;                 // first of the lane's CX columns
    const int y0 = blockIdx.y * R;
    const int c0 = blockIdx.z * g.cg;
    int c1 = c0 + g.cg; if (c1 > g.C) c1 = g.C;
    T acc[R][CX];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int j = 0; j < CX; j++) acc[r][j] = T(0);
    for (int c = c0 + wave; c < c1; c += NW) {
        T wt[KH][KW];
        const T* wc = w + (int64_t)c * (KH * KW);
#pragma unroll
        for (int ky = 0; ky < KH; ky++)
#pragma unroll
            for (int kx = 0; kx < KW; kx++) wt[ky][kx] = wc[ky * KW + kx];
        const T* plane = in + (int64_t)c * g.H * g.W;
        T v[R + KH - 1][CX + KW - 1];
#pragma unroll
        for (int yy = 0; yy < R + KH - 1; yy++) {                // all loads of the window first: one wait for the lot
            load_cols(row_of(plane, y0 + yy, g.W, y0 + yy < g.H), x, v[yy]);
            request_right<KW - 1>(v[yy], row_of(plane, y0 + yy, g.W, y0 + yy < g.H), x, lane);
        }
#pragma unroll
        for (int yy = 0; yy < R + KH - 1; yy++) shift_in_right<KW - 1>(v[yy]);
#pragma unroll
        for (int yy = 0; yy < R + KH - 1; yy++)
#pragma unroll
            for (int ky = 0; ky < KH; ky++) {
                const int r = yy - ky;
                if (r >= 0 && r < R) {
#pragma unroll
                    for (int j = 0; j < CX; j++)
#pragma unroll
                        for (int kx = 0; kx < KW; kx++) acc[r][j] = fused_mad(v[yy][j + kx], wt[ky][kx], acc[r][j]);
                }
            }
    }
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int j = 0; j < CX; j++) red[wave][r][lane * CX + j] = acc[r][j];
    __syncthreads();
    T* dst = partial + (int64_t)blockIdx.z * g.OH * g.OW;
    for (int e = threadIdx.x; e < R * COLS; e += NW * 64) {
        const int r = e / COLS, col = e - r * COLS;
        const int yo = y0 + r, xo = blockIdx.x * COLS + col;
        if (yo < g.OH && xo < g.OW) {
            T s = red[0][r][col];
#pragma unroll
            for (int k = 1; k < NW; k++) s = s + red[k][r][col];
            dst[(int64_t)yo * g.OW + xo] = s;
        }
    }
}

// forward on planes too small for the strips above to fill the machine: a block owns a tile of TR output rows x 64
// columns and reduces ALL channels for it, so the result leaves in one launch with no partial planes.  Its NW
// wavefronts take every NW-th channel.  A wavefront stages a channel's (TR + K - 1) x (64 + K - 1) input window in
// its own piece of LDS with 16-byte loads that run along the rows (the next channel's loads are in flight while the
// current one is multiplied), then every lane reads the K x (TR + K - 1) values above its own output column and
// multiplies them in: the only vector instructions besides the multiply-adds are the LDS accesses.  The tiles of an
// XCD form a band of neighbouring strips, so the K - 1 rows two strips share meet in that XCD's L2 and are
// fetched from memory once.
template <typename T, int K, int TR, int NW>
__global__ __launch_bounds__(NW * 64) void conv_chan_fwd_tiles(ChanArgs g, int col_tiles, int n_tiles, int per_xcd,
                                                               const T* __restrict__ in, const T* __restrict__ w, T* __restrict__ out) {
    constexpr int VEC = 16 / (int)sizeof(T);
    constexpr int WR = TR + K - 1;                               // window rows
    constexpr int PITCH = (64 + K - 1 + VEC - 1) / VEC * VEC;    // window columns, a whole number of 16-byte pieces
    constexpr int PPR = PITCH / VEC;                             // pieces per window row
    constexpr int PIECES = WR * PPR;
    constexpr int LOADS = (PIECES + 63) / 64;
    constexpr int STAGE = WR * PITCH;
    constexpr int WORDS = NW * STAGE > NW * TR * 64 ? NW * STAGE : NW * TR * 64;
    __shared__ __attribute__((aligned(16))) T lds[WORDS];        // the windows; afterwards the wavefronts' sums
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    // blocks are dealt round-robin to the 8 XCDs: XCD k works through tiles [k * per_xcd, (k + 1) * per_xcd)
    const int tile = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if (tile >= n_tiles) return;                                 // whole blocks leave together
    const int x0 = (tile % col_tiles) * 64, y0 = (tile / col_tiles) * TR;
    T* mine = lds + wave * STAGE;

    // piece k of the lane: where it comes from in the plane and where it goes in the window
    unsigned src_off[LOADS];
    int dst_at[LOADS];
#pragma unroll
    for (int k = 0; k < LOADS; k++) {
        const int p = lane + 64 * k;
        const int row = p / PPR, col = (p - row * PPR) * VEC;
        src_off[k] = (unsigned)(((y0 + row) * g.W + x0 + col) * (int)sizeof(T));
        dst_at[k] = p < PIECES ? row * PITCH + col : -1;
    }
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    u32x4 piece[LOADS];
    const unsigned plane_bytes = (unsigned)g.H * (unsigned)g.W * (unsigned)sizeof(T);
    auto request = [&](int c) {                                  // rows past the plane read as zero (range check per dword)
        const BufRsrc plane = buffer_of(in + (int64_t)c * g.H * g.W, plane_bytes);
#pragma unroll
        for (int k = 0; k < LOADS; k++)
            if (LOADS * 64 == PIECES || dst_at[k] >= 0)
                piece[k] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(plane, src_off[k], 0, 0));
    };
    T acc[TR];
#pragma unroll
    for (int r = 0; r < TR; r++) acc[r] = T(0);
    // One channel ahead: the next window's loads are in flight while the current one is multiplied.  (More channels
    // in flight measured slower: 7.1 us with one, 7.4 with two, 7.7 with four on [64,256,256] x [64,5,5].)
    if (wave < g.C) request(wave);
    for (int c = wave; c < g.C; c += NW) {
#pragma unroll
        for (int k = 0; k < LOADS; k++)
            if (LOADS * 64 == PIECES || dst_at[k] >= 0) *(u32x4*)(mine + dst_at[k]) = piece[k];
        __builtin_amdgcn_wave_barrier();                         // LDS operations of a wavefront complete in order
        if (c + NW < g.C) request(c + NW);
        T wt[K][K];
        const T* wc = w + (int64_t)c * (K * K);
#pragma unroll
        for (int ky = 0; ky < K; ky++)
#pragma unroll
            for (int kx = 0; kx < K; kx++) wt[ky][kx] = wc[ky * K + kx];
#pragma unroll
        for (int rr = 0; rr < WR; rr++) {
            T v[K];
#pragma unroll
            for (int kx = 0; kx < K; kx++) v[kx] = mine[rr * PITCH + lane + kx];
#pragma unroll
            for (int ky = 0; ky < K; ky++) {
                const int r = rr - ky;
                if (r >= 0 && r < TR) {
#pragma unroll
                    for (int kx = 0; kx < K; kx++) acc[r] = fused_mad(v[kx], wt[ky][kx], acc[r]);
                }
            }
        }
        __builtin_amdgcn_wave_barrier();                         // the window is read before the next one overwrites it
    }
    __syncthreads();                                             // every wavefront is done with its window
#pragma unroll
    for (int r = 0; r < TR; r++) lds[(wave * TR + r) * 64 + lane] = acc[r];
    __syncthreads();
    for (int e = threadIdx.x; e < TR * 64; e += NW * 64) {       // wavefronts added in a fixed order
        const int r = e >> 6, col = e & 63;
        const int yo = y0 + r, xo = x0 + col;
        if (yo < g.OH && xo < g.OW) {
            T s = lds[r * 64 + col];
#pragma unroll
            for (int k = 1; k < NW; k++) s = s + lds[(k * TR + r) * 64 + col];
            out[(int64_t)yo * g.OW + xo] = s;
        }
    }
}

// gradient w.r.t. the big operand: dx[c][y][x] = sum_ky sum_kx w[c][ky][kx] * err[y-ky][x-kx] (zero outside err)
// wave -> (column block over W, strip of R rows of dx, channel group); the err window of the strip is loaded once
// (one 16-byte load per row) and reused by every channel of the group.  
template <typename T, int KH, int KW, int R>
__global__ __launch_bounds__(256) void conv_chan_dx(ChanArgs g, const T* __restrict__ err, const T* __restrict__ w, T* __restrict__ dx) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int x = blockIdx.x * WAVE_COLS + lane * CX;
    const int y0 = (blockIdx.y * 4 + wave) * R;
    if (y0 >= g.H) return;                                        // whole wavefronts leave together
    const int c0 = blockIdx.z * g.cg;
    int c1 = c0 + g.cg; if (c1 > g.C) c1 = g.C;
    err += (int64_t)c0 * g.err_plane;                             // one error plane per channel: groups of one channel
    // E[rr][i] = err[y0 - (KH-1) + rr][x - (KW-1) + i], zero outside err
    T E[R + KH - 1][CX + KW - 1];
#pragma unroll
    for (int rr = 0; rr < R + KH - 1; rr++) {
        const int ey = y0 - (KH - 1) + rr;
        load_cols(row_of(err, ey, g.OW, ey >= 0 && ey < g.OH), x, &E[rr][KW - 1]);
        request_left<KW - 1>(E[rr], row_of(err, ey, g.OW, ey >= 0 && ey < g.OH), x, lane);
    }
#pragma unroll
    for (int rr = 0; rr < R + KH - 1; rr++) shift_in_left<KW - 1>(E[rr]);
    const bool stores = x < g.W;
    const bool vec_ok = x + CX <= g.W;
    for (int c = c0; c < c1; c++) {
        const T* wc = w + (int64_t)c * g.tap_plane;
        T wt[KH][KW];
#pragma unroll
        for (int ky = 0; ky < KH; ky++)
#pragma unroll
            for (int kx = 0; kx < KW; kx++) wt[ky][kx] = wc[ky * KW + kx];
        T* plane = dx + (int64_t)c * g.H * g.W;
#pragma unroll
        for (int r = 0; r < R; r++) {
            T acc[CX];
#pragma unroll
            for (int j = 0; j < CX; j++) acc[j] = T(0);
#pragma unroll
            for (int ky = 0; ky < KH; ky++)
#pragma unroll
                for (int kx = 0; kx < KW; kx++)
#pragma unroll
                    for (int j = 0; j < CX; j++) acc[j] = fused_mad(E[r + KH - 1 - ky][j - kx + KW - 1], wt[ky][kx], acc[j]);
            if (stores && y0 + r < g.H) {
                T* dst = plane + (int64_t)(y0 + r) * g.W + x;
                if (vec_ok) {
                    store_cols(dst, acc);
                } else {
#pragma unroll
                    for (int j = 0; j < CX; j++) if (x + j < g.W) dst[j] = acc[j];
                }
            }
        }
    }
}

// gradient w.r.t. the taps: dk[c][ky][kx] = sum_y sum_x in[c][y+ky][x+kx] * err[y][x]
//   = sum over input elements (yy, xx) of in[c][yy][xx] * err[yy-ky][xx-kx]
// wave -> (column block over W, strip of S input rows, channel).  The strip is worked off in chunks of R
// rows: the chunk's R input rows and the R + KH - 1 err rows around them are requested (one 16-byte load per
// lane and row) before the first multiply-add, then every input element is multiplied into the KH*KW
// accumulators with statically indexed registers.  Lanes are reduced with wavefront shuffles, strips by a second pass.
template <typename T, int KH, int KW, int R>
__global__ __launch_bounds__(256) void conv_chan_dk(ChanArgs g, int S, int nstrips, const T* __restrict__ in, const T* __restrict__ err, T* __restrict__ partial) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int strip = blockIdx.y * 4 + wave;
    if (strip >= nstrips) return;                                 // whole wavefronts leave together
    const int xx = blockIdx.x * WAVE_COLS + lane * CX;
    const int yy0 = strip * S;
    int yy1 = yy0 + S; if (yy1 > g.H) yy1 = g.H;
    const int c = blockIdx.z;
    T acc[KH][KW];
#pragma unroll
    for (int ky = 0; ky < KH; ky++)
#pragma unroll
        for (int kx = 0; kx < KW; kx++) acc[ky][kx] = T(0);
    const T* plane = in + (int64_t)c * g.H * g.W;
    err += (int64_t)c * g.err_plane;
    for (int y = yy0; y < yy1; y += R) {
        T E[R + KH - 1][CX + KW - 1];                             // E[rr][i] = err[y - (KH-1) + rr][xx - (KW-1) + i], zero outside err
        T V[R][CX];                                               // V[r] = input row y + r, zero past the strip
#pragma unroll
        for (int r = 0; r < R; r++) load_cols(row_of(plane, y + r, g.W, y + r < yy1), xx, V[r]);
#pragma unroll
        for (int rr = 0; rr < R + KH - 1; rr++) {
            const int ey = y - (KH - 1) + rr;
            load_cols(row_of(err, ey, g.OW, ey >= 0 && ey < g.OH), xx, &E[rr][KW - 1]);
            request_left<KW - 1>(E[rr], row_of(err, ey, g.OW, ey >= 0 && ey < g.OH), xx, lane);
        }
#pragma unroll
        for (int rr = 0; rr < R + KH - 1; rr++) shift_in_left<KW - 1>(E[rr]);
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int ky = 0; ky < KH; ky++)
#pragma unroll
                for (int kx = 0; kx < KW; kx++)
#pragma unroll
                    for (int j = 0; j < CX; j++) acc[ky][kx] = fused_mad(V[r][j], E[r - ky + KH - 1][j - kx + KW - 1], acc[ky][kx]);
    }
    // lanes -> lane 63 with data-parallel-primitive adds
    const int part = strip * gridDim.x + blockIdx.x;
#pragma unroll
    for (int ky = 0; ky < KH; ky++)
#pragma unroll
        for (int kx = 0; kx < KW; kx++) acc[ky][kx] = wave_sum_in_lane63(acc[ky][kx]);
    if (lane == 63) {
        T* dst = partial + ((int64_t)part * g.C + c) * (KH * KW);
#pragma unroll
        for (int ky = 0; ky < KH; ky++)
#pragma unroll
            for (int kx = 0; kx < KW; kx++) dst[ky * KW + kx] = acc[ky][kx];
    }
}

// The same sums for planes small enough that the channels alone fill the machine: a block is NW wavefronts of one
// channel that own neighbouring strips; their lanes are reduced with data-parallel-primitive adds, the wavefronts
// through LDS in a fixed order, and the block writes the channel's KH*KW results -- one launch, no partial sums.
// (For larger planes the same blocks with their partial sums joined by the block that draws a channel's last
// ticket were measured: the agent-scope release before the ticket costs more than a second launch, 14.6 us
// against 11.8 on [64,256,256] x [64,5,5]; blocks of eight wavefronts plus a second launch were no faster than
// the strips of conv_chan_dk either.)
template <typename T, int KH, int KW, int R, int NW>
__global__ __launch_bounds__(NW * 64) void conv_chan_dk_joined(ChanArgs g, int S, int nstrips, const T* __restrict__ in, const T* __restrict__ err,
                                                               T* __restrict__ dst) {
    constexpr int KK = KH * KW;
    __shared__ T red[NW][KK];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int strip = blockIdx.y * NW + wave;
    const int xx = blockIdx.x * WAVE_COLS + lane * CX;
    const int yy0 = strip * S;
    int yy1 = yy0 + S; if (yy1 > g.H) yy1 = g.H;
    const int c = blockIdx.z;
    T acc[KH][KW];
#pragma unroll
    for (int ky = 0; ky < KH; ky++)
#pragma unroll
        for (int kx = 0; kx < KW; kx++) acc[ky][kx] = T(0);
    const T* plane = in + (int64_t)c * g.H * g.W;
    for (int y = yy0; y < yy1; y += R) {                          // no trip for a wavefront past the last strip
        T E[R + KH - 1][CX + KW - 1];                             // E[rr][i] = err[y - (KH-1) + rr][xx - (KW-1) + i], zero outside err
        T V[R][CX];                                               // V[r] = input row y + r, zero past the strip
#pragma unroll
        for (int r = 0; r < R; r++) load_cols(row_of(plane, y + r, g.W, y + r < yy1), xx, V[r]);
#pragma unroll
        for (int rr = 0; rr < R + KH - 1; rr++) {
            const int ey = y - (KH - 1) + rr;
            load_cols(row_of(err, ey, g.OW, ey >= 0 && ey < g.OH), xx, &E[rr][KW - 1]);
            request_left<KW - 1>(E[rr], row_of(err, ey, g.OW, ey >= 0 && ey < g.OH), xx, lane);
        }
#pragma unroll
        for (int rr = 0; rr < R + KH - 1; rr++) shift_in_left<KW - 1>(E[rr]);
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int ky = 0; ky < KH; ky++)
#pragma unroll
                for (int kx = 0; kx < KW; kx++)
#pragma unroll
                    for (int j = 0; j < CX; j++) acc[ky][kx] = fused_mad(V[r][j], E[r - ky + KH - 1][j - kx + KW - 1], acc[ky][kx]);
    }
#pragma unroll
    for (int ky = 0; ky < KH; ky++)
#pragma unroll
        for (int kx = 0; kx < KW; kx++) acc[ky][kx] = wave_sum_in_lane63(acc[ky][kx]);
    if (lane == 63) {
#pragma unroll
        for (int ky = 0; ky < KH; ky++)
#pragma unroll
            for (int kx = 0; kx < KW; kx++) red[wave][ky * KW + kx] = acc[ky][kx];
    }
    __syncthreads();
    if (wave != 0) return;                                        // KK <= 64: the first wavefront finishes
    const int t = lane;
    T s = T(0);
    if (t < KK) {
#pragma unroll
        for (int k = 0; k < NW; k++) s = s + red[k][t];           // wavefronts in order
    }
    if (t < KK) dst[(int64_t)c * KK + t] = s;
}

static bool dense_rm(const Cfg& c, int rank) {
    int64_t prod = 1;
    for (int k = rank - 1; k >= 0; k--) {
        if (c.offset[k] != 0) return false;
        if (c.shape[k] > 1 && (c.strides[k] != prod || c.imap[k] != prod || c.spread[k] != 1)) return false;
        prod *= c.shape[k];
    }
    return true;
}

// channel groups: as few channels per group as it takes to put about `want` wavefronts on the machine
static int channels_per_group(int C, int64_t waves_per_group_set, int64_t want) {
    int64_t groups = (want + waves_per_group_set - 1) / waves_per_group_set;
    if (groups < 1) groups = 1;
    if (groups > C) groups = C;
    return (int)((C + groups - 1) / groups);
}

// 2-D valid cross-correlation of large images, square taps: the register-window scheme of the channel kernels
// for one plane.  A wavefront owns R output rows x 256 columns, loads the R + KH - 1 window rows once and reuses
// them for every tap.  For an output element the contributions arrive with ky ascending and kx ascending inside,
// and every product is rounded before it is added (no fused multiply-add): the summation order of
// SimpleCPUConvolution, so the result is bit-identical to conv2d_direct's.
template <typename T, int KH, int KW, int R>
__global__ __launch_bounds__(256) void conv2d_window(int H, int W, const T* __restrict__ img, const T* __restrict__ taps,
                                                     T* __restrict__ out) {
    const int OH = H - KH + 1, OW = W - KW + 1;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int x = blockIdx.x * WAVE_COLS + lane * CX;
    const int y0 = (blockIdx.y * 4 + wave) * R;
    if (y0 >= OH) return;                                        // whole wavefronts leave together
    const T* plane = img + (int64_t)blockIdx.z * H * W;
    T wt[KH][KW];
#pragma unroll
    for (int ky = 0; ky < KH; ky++)
#pragma unroll
        for (int kx = 0; kx < KW; kx++) wt[ky][kx] = taps[ky * KW + kx];
    T v[R + KH - 1][CX + KW - 1];
#pragma unroll
    for (int yy = 0; yy < R + KH - 1; yy++) {
        load_cols(row_of(plane, y0 + yy, W, y0 + yy < H), x, v[yy]);
        request_right<KW - 1>(v[yy], row_of(plane, y0 + yy, W, y0 + yy < H), x, lane);
    }
#pragma unroll
    for (int yy = 0; yy < R + KH - 1; yy++) shift_in_right<KW - 1>(v[yy]);
    T acc[R][CX];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int j = 0; j < CX; j++) acc[r][j] = T(0);
#pragma unroll
    for (int yy = 0; yy < R + KH - 1; yy++)
#pragma unroll
        for (int ky = 0; ky < KH; ky++) {
            const int r = yy - ky;
            if (r >= 0 && r < R) {
#pragma unroll
                for (int j = 0; j < CX; j++)
#pragma unroll
                    for (int kx = 0; kx < KW; kx++) {
                        const T prod = v[yy][j + kx] * wt[ky][kx];
                        acc[r][j] = acc[r][j] + prod;
                    }
            }
        }
    T* dst = out + (int64_t)blockIdx.z * OH * OW;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int yo = y0 + r;
        if (yo < OH) {
            T* p = dst + (int64_t)yo * OW + x;
            if (x + CX <= OW) {
                write_cols(p, acc[r]);
            } else {
#pragma unroll
                for (int j = 0; j < CX; j++) if (x + j < OW) p[j] = acc[r][j];
            }
        }
    }
}

// run-time tap extents -> the template instantiations that exist; false when there is none
template <typename F>
static bool for_taps(int KH, int KW, F&& f) {
    if (KH != KW) return false;
    switch (KH) {
        case 2: f(std::integral_constant<int, 2>{}); return true;
        case 3: f(std::integral_constant<int, 3>{}); return true;
        case 4: f(std::integral_constant<int, 4>{}); return true;
        case 5: f(std::integral_constant<int, 5>{}); return true;
        case 7: f(std::integral_constant<int, 7>{}); return true;
        default: return false;
    }
}

// the three channel kernels for dense f32 or f64 operands; returns NK_OK with *taken = true when one was launched.
// A double takes two registers, so the f64 instantiations work on half as many rows per wavefront.
template <typename T>
static int conv_channel_paths(Device* dev, int d, T* out, const Cfg& c0, const T* s1, const Cfg& c1,
                              const T* s2, const Cfg& c2, bool* taken, bool one_plane = false) {
    constexpr bool F32 = sizeof(T) == 4;
    *taken = false;
    constexpr long waves_per_cu = 8;
    const int64_t want_waves = (int64_t)dev->props.multiProcessorCount * waves_per_cu;
    for (const Cfg* c : {&c0, &c1, &c2})          // a plane is addressed with 32-bit byte offsets; grid y and z are 16-bit
        if ((int64_t)c->shape[1] * c->shape[2] * (int64_t)sizeof(T) >= (int64_t(1) << 31) || c->shape[0] > 65535 || c->shape[1] > 65535) return NK_OK;
    if (d < 0 && c0.shape[0] == 1 && c1.shape[0] == c2.shape[0] && c1.shape[0] > 1) {
        const bool a_big = c1.shape[1] >= c2.shape[1] && c1.shape[2] >= c2.shape[2];
        const bool b_big = c2.shape[1] >= c1.shape[1] && c2.shape[2] >= c1.shape[2];
        if (!a_big && !b_big) return NK_OK;
        const Cfg& big = a_big ? c1 : c2;
        const Cfg& small = a_big ? c2 : c1;
        const T* bigp = a_big ? s1 : s2;
        const T* smallp = a_big ? s2 : s1;
        ChanArgs g{};
        g.C = big.shape[0]; g.H = big.shape[1]; g.W = big.shape[2];
        g.OH = g.H - small.shape[1] + 1; g.OW = g.W - small.shape[2] + 1;
        const int cus = dev->props.multiProcessorCount;
        int rc = NK_OK;
        bool tiled = false;
        const bool ok = for_taps(small.shape[1], small.shape[2], [&](auto K) {
            constexpr int KK = decltype(K)::value;
            g.col_blocks = (g.OW + WAVE_COLS - 1) / WAVE_COLS;
            // Preferred: one block of 16 wavefronts reduces all channels of its (column block, R rows) itself -- no
            // second pass -- when the plane is large enough to give every compute unit such a block (with short strips the
            // window rows a block loads twice outweigh the saved pass: measured on [64,256,256]).
            int tall_r = 0;
            if (g.C >= 16)
                for (int r : {8, 4})
                    if ((F32 || r == 4) && (int64_t)g.col_blocks * ((g.OH + r - 1) / r) >= cus) { tall_r = r; break; }
            if (tall_r) {
                g.cg = g.C;
                dim3 grid(g.col_blocks, (g.OH + tall_r - 1) / tall_r, 1);
                if constexpr (F32) {
                    if (tall_r == 8) hipLaunchKernelGGL((conv_chan_fwd<T, KK, KK, 8, 16>), grid, dim3(1024), 0, dev->stream, g, bigp, smallp, out);
                    else             hipLaunchKernelGGL((conv_chan_fwd<T, KK, KK, 4, 16>), grid, dim3(1024), 0, dev->stream, g, bigp, smallp, out);
                } else {            // eight wavefronts: 256 registers each for the window, 64 KiB of LDS for their sums
                    hipLaunchKernelGGL((conv_chan_fwd<T, KK, KK, 4, 8>), grid, dim3(512), 0, dev->stream, g, bigp, smallp, out);
                }
                return;
            }
            // Planes that still give about one (TR rows x 64 columns) tile per compute unit: every block reduces all
            // channels of its tile, one launch.
            {
                constexpr int NW = F32 ? 16 : 8;
                const int col_tiles = (g.OW + 63) / 64;
                int tr = 0;
                for (int r : {8, 4})
                    if ((int64_t)col_tiles * ((g.OH + r - 1) / r) * 10 >= (int64_t)cus * 9) { tr = r; break; }
                if (!tr && (int64_t)col_tiles * ((g.OH + 3) / 4) * 2 >= cus) tr = 4;
                if (tr && g.C >= NW) {
                    const int n_tiles = col_tiles * ((g.OH + tr - 1) / tr);
                    const int per_xcd = (n_tiles + 7) / 8;
                    g.cg = g.C;
                    if (tr == 8) hipLaunchKernelGGL((conv_chan_fwd_tiles<T, KK, 8, NW>), dim3(8 * per_xcd), dim3(NW * 64), 0, dev->stream, g, col_tiles, n_tiles, per_xcd, bigp, smallp, out);
                    else         hipLaunchKernelGGL((conv_chan_fwd_tiles<T, KK, 4, NW>), dim3(8 * per_xcd), dim3(NW * 64), 0, dev->stream, g, col_tiles, n_tiles, per_xcd, bigp, smallp, out);
                    tiled = true;
                    return;
                }
            }
            // Small planes: parallelism has to come from the channels.  Blocks of four wavefronts take groups of
            // channels (multiples of 4), a second pass adds the partial planes in a fixed order.
            constexpr int R = F32 ? 8 : 4;
            const int strips = (g.OH + R - 1) / R;
            g.cg = channels_per_group(g.C, (int64_t)g.col_blocks * strips * 4, want_waves);
            g.cg = (g.cg + 3) / 4 * 4;
            const int groups = (g.C + g.cg - 1) / g.cg;
            void* ws = nullptr;
            const int on = g.OH * g.OW;
            if ((rc = workspace(dev, (uint64_t)groups * on * sizeof(T), &ws))) return;
            dim3 grid(g.col_blocks, strips, groups);
            hipLaunchKernelGGL((conv_chan_fwd<T, KK, KK, R, 4>), grid, dim3(256), 0, dev->stream, g, bigp, smallp, groups == 1 ? out : (T*)ws);
            if (groups > 1)
                hipLaunchKernelGGL(conv_partial_reduce<T>, dim3((on + 255) / 256), dim3(256), 0, dev->stream, groups, on, (const T*)ws, out);
        });
        if (!ok) return NK_OK;
        if (rc) return rc;
        NK_HIP(hipGetLastError());
        set_path(tiled ? "chan_fwd_tiles" : "chan_fwd");
        *taken = true;
        return NK_OK;
    }
    // gradients, src2 = the error: one plane [1,OH,OW] shared by the channels of [C,H,W] x [C,k,k], or -- a batch of
    // images under one set of taps, [B,H,W] x [1,k,k] -- one plane per image [B,OH,OW]
    const bool shared_err = c2.shape[0] == 1 && c0.shape[0] == c1.shape[0] && (c0.shape[0] > 1 || one_plane);
    const bool batch_dx = c2.shape[0] > 1 && c0.shape[0] == c2.shape[0] && c1.shape[0] == 1;
    const bool batch_dk = c2.shape[0] > 1 && c1.shape[0] == c2.shape[0] && c0.shape[0] == 1;
    if (d >= 0 && (shared_err || batch_dx || batch_dk)) {
        const int OH = c2.shape[1], OW = c2.shape[2];
        // dx: the drain is the big operand, src1 the taps
        if ((shared_err || batch_dx) && c0.shape[1] == OH + c1.shape[1] - 1 && c0.shape[2] == OW + c1.shape[2] - 1 &&
            (c0.shape[1] > c1.shape[1] || c1.shape[1] == 1) && (c0.shape[2] > c1.shape[2] || c1.shape[2] == 1)) {
            constexpr int R = 4;
            ChanArgs g{};
            g.C = c0.shape[0]; g.H = c0.shape[1]; g.W = c0.shape[2]; g.OH = OH; g.OW = OW;
            const int strips = (g.H + R - 1) / R;
            const bool ok = for_taps(c1.shape[1], c1.shape[2], [&](auto K) {
                constexpr int KK = decltype(K)::value;
                g.col_blocks = (g.W + WAVE_COLS - 1) / WAVE_COLS;
                g.err_plane = batch_dx ? OH * OW : 0;
                g.tap_plane = batch_dx ? 0 : KK * KK;
                g.cg = channels_per_group(g.C, (int64_t)g.col_blocks * strips, want_waves);
                if (g.cg < 2 && g.C >= 2) g.cg = 2;          // amortise the err window over at least two channels
                if (batch_dx) g.cg = 1;                      // every image has its own err window
                const int groups = (g.C + g.cg - 1) / g.cg;
                dim3 grid(g.col_blocks, (strips + 3) / 4, groups);
                hipLaunchKernelGGL((conv_chan_dx<T, KK, KK, R>), grid, dim3(256), 0, dev->stream, g, s2, s1, out);
            });
            if (!ok) return NK_OK;
            NK_HIP(hipGetLastError());
            set_path("chan_dx");
            *taken = true;
            return NK_OK;
        }
        // dk: the drain is the taps, src1 the big operand
        if ((shared_err || batch_dk) && c1.shape[1] == OH + c0.shape[1] - 1 && c1.shape[2] == OW + c0.shape[2] - 1 && c0.shape[1] < c1.shape[1] && c0.shape[2] < c1.shape[2]) {
            ChanArgs g{};
            g.err_plane = batch_dk ? OH * OW : 0;
            g.C = c1.shape[0]; g.H = c1.shape[1]; g.W = c1.shape[2]; g.OH = OH; g.OW = OW;
            g.cg = 1;
            constexpr int R = F32 ? 8 : 4;
            int rc = NK_OK;
            const bool ok = for_taps(c0.shape[1], c0.shape[2], [&](auto K) {
                constexpr int KK = decltype(K)::value;
                g.col_blocks = (g.W + WAVE_COLS - 1) / WAVE_COLS;
                // rows per strip: enough strips for the machine, a whole number of R-row chunks each
                int64_t strips = (want_waves + (int64_t)g.col_blocks * g.C - 1) / ((int64_t)g.col_blocks * g.C);
                if (strips < 1) strips = 1;
                int S = (int)((g.H + strips - 1) / strips);
                S = (S + R - 1) / R * R;
                const int nstrips = (g.H + S - 1) / S;
                const int parts = nstrips * g.col_blocks;
                const int on = g.C * KK * KK;
                void* ws = nullptr;
                constexpr int NW = 8;
                if (!batch_dk && g.col_blocks == 1 && nstrips <= NW) {
                    // a channel fits one block of NW wavefronts: finished in one launch
                    dim3 grid(1, 1, g.C);
                    hipLaunchKernelGGL((conv_chan_dk_joined<T, KK, KK, R, NW>), grid, dim3(NW * 64), 0, dev->stream, g, S, nstrips, s1, s2, out);
                    return;
                }
                if ((rc = workspace(dev, (uint64_t)parts * on * sizeof(T), &ws))) return;
                dim3 grid(g.col_blocks, (nstrips + 3) / 4, g.C);
                hipLaunchKernelGGL((conv_chan_dk<T, KK, KK, R>), grid, dim3(256), 0, dev->stream, g, S, nstrips, s1, s2, (T*)ws);
                // a batch sums the images' tap gradients as well: [parts][C][k*k] read as [parts * C][k*k]
                const int sums = batch_dk ? parts * g.C : parts, outs = batch_dk ? KK * KK : on;
                hipLaunchKernelGGL(conv_partial_reduce_wide<T>, dim3((outs + 3) / 4), dim3(256), 0, dev->stream, sums, outs, (const T*)ws, out);
            });
            if (!ok) return NK_OK;
            if (rc) return rc;
            NK_HIP(hipGetLastError());
            set_path("chan_dk");
            *taken = true;
            return NK_OK;
        }
    }
    return NK_OK;
}

// Forward 2-D convolution of dense row-major operands with one set of taps, [H,W] x [kh,kw] or
// [B,H,W] x [1,kh,kw]: the case the reference's CPU device hands to SimpleCPUConvolution
// (J/backend/main/implementations/convolution/AbstractCPUConvolution.java:18-23, SimpleCPUConvolution.java:143-159).
// One thread per output element, taps through scalar loads, the sum in that class's order (ky outer, kx inner,
// product rounded before the add): bit-identical to it in f32 and f64.
template <typename T>
__global__ __launch_bounds__(256) void conv2d_direct(int B, int H, int W, int KH, int KW, const T* __restrict__ img,
                                                     const T* __restrict__ taps, T* __restrict__ out) {
    const int OH = H - KH + 1, OW = W - KW + 1;
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= B * OH * OW) return;
    const int b = idx / (OH * OW);
    const int rem = idx - b * (OH * OW);
    const int y = rem / OW, x = rem - y * OW;
    const T* p = img + ((int64_t)b * H + y) * W + x;
    T sum = T(0);
    for (int ky = 0; ky < KH; ky++)
        for (int kx = 0; kx < KW; kx++) {
            const T prod = p[ky * W + kx] * taps[ky * KW + kx];
            sum = sum + prod;
        }
    out[idx] = sum;
}

template <typename T>
static bool conv2d_direct_path(Device* dev, int d, int rank, T* out, const Cfg& c0, const T* s1, const Cfg& c1, const T* s2, const Cfg& c2) {
    if (d >= 0 || (rank != 2 && rank != 3)) return false;
    if (!dense_rm(c0, rank) || !dense_rm(c1, rank) || !dense_rm(c2, rank)) return false;
    const int o = rank - 2;
    const bool a_img = c1.shape[o] >= c2.shape[o] && c1.shape[o + 1] >= c2.shape[o + 1];
    const bool b_img = c2.shape[o] >= c1.shape[o] && c2.shape[o + 1] >= c1.shape[o + 1];
    if (!a_img && !b_img) return false;
    const Cfg& img = a_img ? c1 : c2;
    const Cfg& tap = a_img ? c2 : c1;
    if (rank == 3 && tap.shape[0] != 1) return false;
    const int B = rank == 3 ? (int)img.shape[0] : 1;
    const int64_t n = (int64_t)B * (img.shape[o] - tap.shape[o] + 1) * (img.shape[o + 1] - tap.shape[o + 1] + 1);
    if (n >= ((int64_t)1 << 31)) return false;
    {
        // large images with square taps: the register-window kernel (same sums, same order); half the rows in f64
        const int H = (int)img.shape[o], W = (int)img.shape[o + 1];
        if (n >= 65536 && (int64_t)H * W * (int64_t)sizeof(T) < ((int64_t)1 << 31) && B <= 65535) {
            constexpr int R = sizeof(T) == 4 ? 8 : 4;
            const int OH = H - (int)tap.shape[o] + 1, OW = W - (int)tap.shape[o + 1] + 1;
            // strips of R rows per wavefront; half as many rows while that still leaves fewer than four wavefronts per
            // SIMD (more wavefronts overlap their loads with the others' arithmetic: [2048,2048] x [5,5] 11.4 -> 10.4 us,
            // [1024,1024] x [5,5] 7.1 -> 4.8 us; [4096,4096] x [3,3] keeps R rows, 22.9 against 24.8 us)
            const int64_t waves_r = (int64_t)((OW + WAVE_COLS - 1) / WAVE_COLS) * ((OH + R - 1) / R) * B;
            const int RR = (sizeof(T) == 4 && waves_r < 16 * (int64_t)dev->props.multiProcessorCount) ? 4 : R;
            const dim3 grid((unsigned)((OW + WAVE_COLS - 1) / WAVE_COLS), (unsigned)(((OH + RR - 1) / RR + 3) / 4), (unsigned)B);
            const T* ip = a_img ? s1 : s2;
            const T* tp = a_img ? s2 : s1;
            if (grid.y <= 65535 && for_taps((int)tap.shape[o], (int)tap.shape[o + 1], [&](auto K) {
                    constexpr int KK = decltype(K)::value;
                    if (RR == 4) hipLaunchKernelGGL((conv2d_window<T, KK, KK, 4>), grid, dim3(256), 0, dev->stream, H, W, ip, tp, out);
                    else hipLaunchKernelGGL((conv2d_window<T, KK, KK, R>), grid, dim3(256), 0, dev->stream, H, W, ip, tp, out);
                })) {
                set_path("simple2d_window");
                return true;
            }
        }
    }
    set_path("simple2d");
    hipLaunchKernelGGL(conv2d_direct<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, dev->stream, B, (int)img.shape[o], (int)img.shape[o + 1],
                       (int)tap.shape[o], (int)tap.shape[o + 1], a_img ? s1 : s2, a_img ? s2 : s1, out);
    return true;
}

// Forward 1-D convolution of dense vectors, out[j] = sum_k x[j + k] * w[k]: a block owns 256 * R neighbouring outputs,
// stages the 256 * R + K - 1 inputs they read in LDS once, and every thread adds its R sums tap by tap (k ascending,
// product rounded before the add) -- the order of _convolve32 / _convolve64 for rank 1, so the result is theirs bit for
// bit.  The taps come through scalar loads (the index is the same for the whole block).
template <typename T, int R>
__global__ __launch_bounds__(256) void conv1d_direct(int N, int K, const T* __restrict__ x, const T* __restrict__ w, T* __restrict__ out) {
    extern __shared__ __attribute__((aligned(16))) unsigned char conv1d_lds[];
    T* tile = (T*)conv1d_lds;
    const int n_out = N - K + 1;
    const int j0 = blockIdx.x * (256 * R);
    const int span = 256 * R + K - 1;
    for (int e = threadIdx.x; e < span; e += 256) tile[e] = j0 + e < N ? x[j0 + e] : T(0);
    __syncthreads();
    T acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = T(0);
    for (int k = 0; k < K; k++) {
        const T wk = w[k];
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = acc[r] + tile[r * 256 + threadIdx.x + k] * wk;
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int j = j0 + r * 256 + (int)threadIdx.x;
        if (j < n_out) out[j] = acc[r];
    }
}

// Gradient of the same convolution by the long operand: dx[i] = sum_e w[i - e] * err[e] over the error entries that
// pass the bounds test, e ascending (_deConvolve32 / _deConvolve64 for rank 1).  The same staging; entries outside the
// error are skipped by a predicate, not replaced by zeros (a zero times an infinite tap would not be nothing).
template <typename T, int R>
__global__ __launch_bounds__(256) void conv1d_grad_long(int N, int K, const T* __restrict__ w, const T* __restrict__ err, T* __restrict__ dx) {
    extern __shared__ __attribute__((aligned(16))) unsigned char conv1d_lds[];
    T* tile = (T*)conv1d_lds;
    const int n_err = N - K + 1;
    const int i0 = blockIdx.x * (256 * R);
    const int first = i0 - (K - 1);                              // error index of tile[0]
    const int span = 256 * R + K - 1;
    for (int s = threadIdx.x; s < span; s += 256) {
        const int e = first + s;
        tile[s] = e >= 0 && e < n_err ? err[e] : T(0);
    }
    __syncthreads();
    T acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = T(0);
    for (int s = 0; s < K; s++) {                                 // tap K - 1 - s meets error entry i - (K - 1) + s
        const T wk = w[K - 1 - s];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int local = r * 256 + (int)threadIdx.x;
            const int e = first + local + s;
            if (e >= 0 && e < n_err) acc[r] = acc[r] + wk * tile[local + s];
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int i = i0 + r * 256 + (int)threadIdx.x;
        if (i < N) dx[i] = acc[r];
    }
}

// ... and by the taps: dk[k] = sum_e x[k + e] * err[e].  Few outputs with long sums: a block takes 1024 entries of the
// error, stages them and the inputs they meet in LDS, thread t adds the partial sums of the taps t, t + 256, ...;
// conv_partial_reduce_wide adds the blocks' partial sums.  The terms are the reference's, their order is not
// (norm-wise 1e-5 / 1e-12, like the other split sums).
constexpr int CONV1D_SEG = 1024;
template <typename T>
__global__ __launch_bounds__(256) void conv1d_grad_taps(int N, int K, const T* __restrict__ x, const T* __restrict__ err, T* __restrict__ partial) {
    extern __shared__ __attribute__((aligned(16))) unsigned char conv1d_lds[];
    T* xt = (T*)conv1d_lds;                                       // CONV1D_SEG + K - 1 inputs
    T* et = xt + CONV1D_SEG + K - 1;                              // CONV1D_SEG error entries
    const int n_err = N - K + 1;
    const int e0 = blockIdx.x * CONV1D_SEG;
    const int count = n_err - e0 < CONV1D_SEG ? n_err - e0 : CONV1D_SEG;
    for (int s = threadIdx.x; s < CONV1D_SEG + K - 1; s += 256) xt[s] = e0 + s < N ? x[e0 + s] : T(0);
    for (int s = threadIdx.x; s < CONV1D_SEG; s += 256) et[s] = s < count ? err[e0 + s] : T(0);
    __syncthreads();
    for (int k = threadIdx.x; k < K; k += 256) {
        T acc = T(0);
        for (int e = 0; e < count; e++) acc = acc + xt[k + e] * et[e];
        partial[(int64_t)blockIdx.x * K + k] = acc;
    }
}

template <typename T>
static bool conv1d_direct_path(Device* dev, int d, int rank, T* out, const Cfg& c0, const T* s1, const Cfg& c1, const T* s2, const Cfg& c2) {
    if (rank != 1 || !dense_rm(c0, 1) || !dense_rm(c1, 1) || !dense_rm(c2, 1)) return false;
    if (d >= 0) {
        // drain = the long operand, src1 = the taps, src2 = the error [N - K + 1]
        if (c0.shape[0] < c1.shape[0]) {
            // drain = the taps [K], src1 = the long operand [N], src2 = the error [N - K + 1]
            const int K = c0.shape[0], N = c1.shape[0], n_err = N - K + 1;
            if (K < 2 || K > 4096 || c2.shape[0] != n_err || n_err < 4096) return false;
            const int parts = (n_err + CONV1D_SEG - 1) / CONV1D_SEG;
            void* ws = nullptr;
            if (workspace(dev, (uint64_t)parts * K * sizeof(T), &ws)) return false;
            const size_t lds = (size_t)(2 * CONV1D_SEG + K - 1) * sizeof(T);
            hipLaunchKernelGGL(conv1d_grad_taps<T>, dim3(parts), dim3(256), lds, dev->stream, N, K, s1, s2, (T*)ws);
            hipLaunchKernelGGL(conv_partial_reduce_wide<T>, dim3((K + 3) / 4), dim3(256), 0, dev->stream, parts, K, (const T*)ws, out);
            set_path("simple1d_grad_taps");
            return true;
        }
        const int N = c0.shape[0], K = c1.shape[0];
        constexpr int R = 4;
        if (K < 2 || K > 4096 || N <= K || c2.shape[0] != N - K + 1 || N < 4096) return false;
        const unsigned blocks = (unsigned)((N + 256 * R - 1) / (256 * R));
        const size_t lds = (size_t)(256 * R + K - 1) * sizeof(T);
        hipLaunchKernelGGL((conv1d_grad_long<T, R>), dim3(blocks), dim3(256), lds, dev->stream, N, K, s1, s2, out);
        set_path("simple1d_grad");
        return true;
    }
    const bool first_long = c1.shape[0] >= c2.shape[0];
    const int N = first_long ? c1.shape[0] : c2.shape[0], K = first_long ? c2.shape[0] : c1.shape[0];
    constexpr int R = 4;
    if (K < 2 || K > 4096 || N - K + 1 < 4096) return false;          // short vectors stay on the general kernel
    const T* x = first_long ? s1 : s2;
    const T* w = first_long ? s2 : s1;
    const unsigned blocks = (unsigned)((N - K + 1 + 256 * R - 1) / (256 * R));
    const size_t lds = (size_t)(256 * R + K - 1) * sizeof(T);
    hipLaunchKernelGGL((conv1d_direct<T, R>), dim3(blocks), dim3(256), lds, dev->stream, N, K, x, w, out);
    set_path("simple1d");
    return true;
}

template <typename T>
static int conv_typed(Device* dev, int d, int rank, nk_buf drn, const Cfg& c0, nk_buf a, const Cfg& c1, nk_buf b,
                      const Cfg& c2, int64_t n) {
    T* out = (T*)drn;
    const T* s1 = (const T*)a;
    const T* s2 = (const T*)b;
    if (conv2d_direct_path<T>(dev, d, rank, out, c0, s1, c1, s2, c2) || conv1d_direct_path<T>(dev, d, rank, out, c0, s1, c1, s2, c2)) {
        NK_HIP(hipGetLastError());
        return NK_OK;
    }
    if constexpr (std::is_floating_point<T>::value) {
        if (rank == 3 && dense_rm(c0, rank) && dense_rm(c1, rank) && dense_rm(c2, rank)) {
            bool taken = false;
            if (int e = conv_channel_paths<T>(dev, d, out, c0, s1, c1, s2, c2, &taken)) return e;
            if (taken) return NK_OK;
        }
        // both gradients of a 2-D image convolution [H,W] x [kh,kw] are the one-channel case of the same kernels
        if (rank == 2 && d >= 0 && dense_rm(c0, rank) && dense_rm(c1, rank) && dense_rm(c2, rank)) {
            auto plane = [](const Cfg& c) { Cfg p{}; p.shape[0] = 1; p.shape[1] = c.shape[0]; p.shape[2] = c.shape[1]; return p; };
            bool taken = false;
            if (int e = conv_channel_paths<T>(dev, d, out, plane(c0), s1, plane(c1), s2, plane(c2), &taken, true)) return e;
            if (taken) return NK_OK;
        }
    }
    ConvArgs A{};
    A.rank = rank; A.n = (unsigned)n; A.c0 = c0; A.c1 = c1; A.c2 = c2;
    // terms of one sum (the gradient's upper bound: all of src2); few long sums go to the kernel that splits them
    int64_t terms = 1;
    for (int k = 0; k < rank; k++) terms *= d < 0 ? (c1.shape[k] < c2.shape[k] ? c1.shape[k] : c2.shape[k]) : c2.shape[k];
    if (d >= 0) {                                  // ... of which only the window that passes the bounds test counts
        int64_t window = 1;
        for (int k = 0; k < rank; k++) window *= c1.shape[k] < c2.shape[k] ? c1.shape[k] : c2.shape[k];
        if (window < terms) terms = window;
    }
    // one thread per drain element feeds the machine only with many elements or short sums; otherwise a wavefront
    // (sums of a few hundred terms) or a block per element, and segments when even that gives too few blocks
    const bool few = n < ((int64_t)1 << 17) && terms >= 128;
    if ((terms >= 1024 && n <= ((int64_t)1 << 18)) || few) {
        const int GS = terms >= 2048 ? 256 : 64;
        const int EPB = 256 / GS;
        const int64_t groups = (n + EPB - 1) / EPB;
        SplitArgs S{};
        S.per_xcd = (unsigned)((groups + 7) / 8);
        int64_t segs = 1;
        if (groups < 1024) {
            segs = (2048 + groups - 1) / groups;
            const int64_t most = terms / ((int64_t)GS * 8);
            if (segs > most) segs = most;
            if (segs > 256) segs = 256;
            if (segs < 1) segs = 1;
        }
        S.seg_terms = (unsigned)((terms + segs - 1) / segs);
        segs = (terms + S.seg_terms - 1) / S.seg_terms;
        void* ws = nullptr;
        if (segs > 1)
            if (int e = workspace(dev, (uint64_t)segs * n * sizeof(T), &ws)) return e;
        set_path(d < 0 ? "split_fwd" : "split_bwd");
        const dim3 grid(8u * S.per_xcd, (unsigned)segs);
        auto go = [&](auto R) {
            constexpr int RANK = decltype(R)::value;
            auto sized = [&](auto gs, auto seg) {
                constexpr int G = decltype(gs)::value;
                constexpr bool SEG = decltype(seg)::value;
                if (d < 0) hipLaunchKernelGGL((conv_split<T, false, RANK, G, SEG>), grid, dim3(256), 0, dev->stream, A, S, out, (T*)ws, s1, s2);
                else       hipLaunchKernelGGL((conv_split<T, true, RANK, G, SEG>), grid, dim3(256), 0, dev->stream, A, S, out, (T*)ws, s1, s2);
            };
            if (GS == 256) { if (segs > 1) sized(std::integral_constant<int, 256>{}, std::true_type{}); else sized(std::integral_constant<int, 256>{}, std::false_type{}); }
            else           { if (segs > 1) sized(std::integral_constant<int, 64>{}, std::true_type{}); else sized(std::integral_constant<int, 64>{}, std::false_type{}); }
        };
        if (rank == 2) go(std::integral_constant<int, 2>{});
        else if (rank == 3) go(std::integral_constant<int, 3>{});
        else if (rank == 4) go(std::integral_constant<int, 4>{});
        else go(std::integral_constant<int, 0>{});
        if (segs > 1)
            hipLaunchKernelGGL(conv_split_finish<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, dev->stream, c0, rank, (unsigned)n, (int)segs, (const T*)ws, out);
        NK_HIP(hipGetLastError());
        return NK_OK;
    }
    unsigned blocks = (unsigned)((n + 255) / 256);
    if (blocks > 65536) blocks = 65536;
    set_path(d < 0 ? "literal_fwd" : "literal_bwd");
    auto go = [&](auto R) {
        constexpr int RANK = decltype(R)::value;
        if (d < 0) hipLaunchKernelGGL((conv_fwd_literal<T, RANK>), dim3(blocks), dim3(256), 0, dev->stream, A, out, s1, s2);
        else       hipLaunchKernelGGL((conv_bwd_literal<T, RANK>), dim3(blocks), dim3(256), 0, dev->stream, A, out, s1, s2);
    };
    if (rank == 2) go(std::integral_constant<int, 2>{});
    else if (rank == 3) go(std::integral_constant<int, 3>{});
    else if (rank == 4) go(std::integral_constant<int, 4>{});
    else go(std::integral_constant<int, 0>{});
    NK_HIP(hipGetLastError());
    return NK_OK;
}

}  // namespace nk

using namespace nk;

extern "C" int nk_convolution(nk_dev h, int d, int dtype, int rank, nk_buf drn, const int32_t* drn_cfg, nk_buf a,
                              const int32_t* a_cfg, nk_buf b, const int32_t* b_cfg, int64_t n) {
    NK_DEVICE(dev, h);
    NK_REQUIRE(dtype == NK_F32 || dtype == NK_F64, "nk_convolution: unknown dtype %d", dtype);
    if (int e = check_cfg("nk_convolution(drain)", drn_cfg, rank)) return e;
    if (int e = check_cfg("nk_convolution(src1)", a_cfg, rank)) return e;
    if (int e = check_cfg("nk_convolution(src2)", b_cfg, rank)) return e;
    int64_t size = 1;
    for (int k = 0; k < rank; k++) size *= drn_cfg[k];
    NK_REQUIRE(n == size && size < ((int64_t)1 << 31), "nk_convolution: n = %lld but the drain holds %lld elements", (long long)n, (long long)size);
    if (d < 0)
        for (int k = 0; k < rank; k++) {
            int diff = a_cfg[k] - b_cfg[k];
            if (diff < 0) diff = -diff;
            // ConvUtil.shapeOfCon (J/backend/main/operations/ConvUtil.java:61-66)
            NK_REQUIRE(drn_cfg[k] == diff + 1, "nk_convolution: drain extent %d on axis %d, expected |%d - %d| + 1", drn_cfg[k], k, a_cfg[k], b_cfg[k]);
        }
    const int eb = dtype_bytes(dtype);
    if (int e = check_extent(dev, "nk_convolution(drain)", drn, drn_cfg, rank, eb)) return e;
    if (int e = check_extent(dev, "nk_convolution(src1)", a, a_cfg, rank, eb)) return e;
    if (int e = check_extent(dev, "nk_convolution(src2)", b, b_cfg, rank, eb)) return e;
    Cfg c0, c1, c2;
    load_cfg(c0, drn_cfg, rank); load_cfg(c1, a_cfg, rank); load_cfg(c2, b_cfg, rank);
    tame_unravel(c0, rank, n);              // (the operands are read at positions derived from the drain's nd-index)
    return dtype == NK_F32 ? conv_typed<float>(dev, d, rank, drn, c0, a, c1, b, c2, n)
                           : conv_typed<double>(dev, d, rank, drn, c0, a, c1, b, c2, n);
}
