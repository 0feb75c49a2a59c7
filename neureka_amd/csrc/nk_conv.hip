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
//   chan_fwd       rank 3, dense row-major, full reduction over axis 0 (channels):
//                  [C,H,W] x [C,kh,kw] -> [1,H-kh+1,W-kw+1].  Channels are split over the four
//                  wavefronts of a block and over `splits` blocks; each wavefront stages its channel's
//                  input halo tile in LDS, the kernel taps sit in LDS too; partial sums are reduced
//                  across wavefronts in LDS and across blocks by a second pass over a scratch buffer.
//   chan_dx        gradient w.r.t. the [C,H,W] operand: per channel a "full" correlation of the error
//                  with that channel's kh x kw taps, error tile + halo staged in LDS.
//   chan_dk        gradient w.r.t. the [C,kh,kw] operand: per (channel, tap) a dot product of the
//                  shifted input plane with the error, block-wide reduction (wavefront shuffles + LDS).
#include "nk_internal.h"

namespace nk {

struct ConvArgs {
    int rank;
    unsigned n;
    Cfg c0, c1, c2;
};

template <typename T>
__global__ __launch_bounds__(256) void conv_fwd_literal(ConvArgs A, T* __restrict__ drn, const T* __restrict__ s1,
                                                        const T* __restrict__ s2) {
    const unsigned step = gridDim.x * blockDim.x;
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < A.n; i += step) {
        int o[NK_MAX_RANK], b1[NK_MAX_RANK], b2[NK_MAX_RANK], j[NK_MAX_RANK], m[NK_MAX_RANK];
        nd_of_flat(A.c0, A.rank, (int)i, o);
        for (int k = 0; k < A.rank; k++) {
            const int e1 = A.c1.shape[k], e2 = A.c2.shape[k];
            b1[k] = e1 >= e2 ? o[k] : 0;
            b2[k] = e1 <= e2 ? o[k] : 0;
            m[k] = e1 < e2 ? e1 : e2;
            j[k] = 0;
        }
        T value = T(0);
        bool running = true;
        while (running) {
            int i1[NK_MAX_RANK], i2[NK_MAX_RANK];
            for (int k = 0; k < A.rank; k++) { i1[k] = b1[k] + j[k]; i2[k] = b2[k] + j[k]; }
            T prod = s1[phys_of_nd(A.c1, A.rank, i1)] * s2[phys_of_nd(A.c2, A.rank, i2)];
            value = value + prod;
            int k = 0;
            for (; k < A.rank; k++) {
                if (++j[k] < m[k]) break;
                j[k] = 0;
            }
            running = k < A.rank;
        }
        drn[phys_of_nd(A.c0, A.rank, o)] = value;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void conv_bwd_literal(ConvArgs A, T* __restrict__ drn, const T* __restrict__ s1,
                                                        const T* __restrict__ s2) {
    const unsigned step = gridDim.x * blockDim.x;
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < A.n; i += step) {
        int o[NK_MAX_RANK], lo[NK_MAX_RANK], hi[NK_MAX_RANK], e[NK_MAX_RANK];
        nd_of_flat(A.c0, A.rank, (int)i, o);
        bool empty = false;
        for (int k = 0; k < A.rank; k++) {
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
            int i1[NK_MAX_RANK];
            for (int k = 0; k < A.rank; k++) i1[k] = A.c0.shape[k] > A.c1.shape[k] ? o[k] - e[k] : o[k] + e[k];
            T prod = s1[phys_of_nd(A.c1, A.rank, i1)] * s2[phys_of_nd(A.c2, A.rank, e)];
            value = value + prod;
            int k = 0;
            for (; k < A.rank; k++) {
                if (++e[k] < hi[k]) break;
                e[k] = lo[k];
            }
            running = k < A.rank;
        }
        drn[phys_of_nd(A.c0, A.rank, o)] = value;
    }
}

// ------------------------------------------------------------------------------------------------
// chan_fwd: out[y][x] = sum_c sum_ky sum_kx in[c][y+ky][x+kx] * w[c][ky][kx]
struct ChanArgs {
    int C, H, W, KH, KW, OH, OW;
    int splits;          // channel groups (blocks along z)
    int cps;             // channels per split
};

constexpr int FT_Y = 16, FT_X = 64;      // output tile of chan_fwd
constexpr int MAX_KH = 8, MAX_KW = 8;

__device__ __forceinline__ void wave_lds_sync() {
    // LDS traffic of one wavefront is processed in order; the fences keep the compiler from moving the
    // accesses across this point, no block-wide barrier is needed for data private to a wavefront
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// TKH/TKW > 0: tap extents known at compile time (the column of the halo a lane needs is kept in
// registers and reused by all ky); 0: run-time extents up to MAX_KH x MAX_KW.
template <typename T, int TKH, int TKW>
__global__ __launch_bounds__(256) void conv_chan_fwd(ChanArgs g, const T* __restrict__ in, const T* __restrict__ w,
                                                     T* __restrict__ partial) {
    constexpr int HP = FT_X + MAX_KW;               // halo pitch in elements
    constexpr int HR = FT_Y + MAX_KH - 1;
    __shared__ T halo[4][HR * HP];
    __shared__ T taps[4][MAX_KH * MAX_KW];
    __shared__ T red[4][FT_Y * FT_X];

    const int KH = TKH ? TKH : g.KH, KW = TKW ? TKW : g.KW;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int x0 = blockIdx.x * FT_X, y0 = blockIdx.y * FT_Y;
    const int c_begin = blockIdx.z * g.cps;
    int c_end = c_begin + g.cps; if (c_end > g.C) c_end = g.C;
    const int hw = FT_X + KW - 1, hh = FT_Y + KH - 1;

    T acc[FT_Y];
#pragma unroll
    for (int r = 0; r < FT_Y; r++) acc[r] = T(0);

    // a lane owns output column x0 + lane for all FT_Y rows of the tile; a wavefront owns every 4th
    // channel of the block's channel group
    for (int c = c_begin + wave; c < c_end; c += 4) {
        const T* plane = in + (int64_t)c * g.H * g.W;
        for (int r = 0; r < hh; r++) {
            const int y = y0 + r;
            for (int xx = lane; xx < hw; xx += 64) {
                const int x = x0 + xx;
                T v = T(0);
                if (y < g.H && x < g.W) v = plane[(int64_t)y * g.W + x];
                halo[wave][r * HP + xx] = v;
            }
        }
        if (lane < KH * KW) taps[wave][lane] = w[(int64_t)c * KH * KW + lane];
        wave_lds_sync();
        if constexpr (TKH > 0) {
#pragma unroll
            for (int kx = 0; kx < TKW; kx++) {
                T col[FT_Y + TKH - 1];
#pragma unroll
                for (int r = 0; r < FT_Y + TKH - 1; r++) col[r] = halo[wave][r * HP + lane + kx];
#pragma unroll
                for (int ky = 0; ky < TKH; ky++) {
                    const T t = taps[wave][ky * TKW + kx];
#pragma unroll
                    for (int r = 0; r < FT_Y; r++) acc[r] = __builtin_fma(col[r + ky], t, acc[r]);
                }
            }
        } else {
            for (int ky = 0; ky < KH; ky++)
                for (int kx = 0; kx < KW; kx++) {
                    const T t = taps[wave][ky * KW + kx];
#pragma unroll
                    for (int r = 0; r < FT_Y; r++) acc[r] = __builtin_fma(halo[wave][(r + ky) * HP + lane + kx], t, acc[r]);
                }
        }
        wave_lds_sync();
    }
    // reduce the four wavefronts
#pragma unroll
    for (int r = 0; r < FT_Y; r++) red[wave][r * FT_X + lane] = acc[r];
    __syncthreads();
    for (int idx = threadIdx.x; idx < FT_Y * FT_X; idx += 256) {
        const int r = idx / FT_X, xx = idx % FT_X;
        const int y = y0 + r, x = x0 + xx;
        if (y < g.OH && x < g.OW) {
            T s = (red[0][idx] + red[1][idx]) + (red[2][idx] + red[3][idx]);
            partial[((int64_t)blockIdx.z * g.OH + y) * g.OW + x] = s;
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void conv_chan_fwd_reduce(int splits, int n, const T* __restrict__ partial, T* __restrict__ out) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    T s = T(0);
    for (int k = 0; k < splits; k++) s = s + partial[(int64_t)k * n + i];
    out[i] = s;
}

// chan_dx: dx[c][y][x] = sum_ky sum_kx w[c][ky][kx] * err[y-ky][x-kx]   (terms with err out of range vanish)
constexpr int DT_Y = 16, DT_X = 64;
template <typename T>
__global__ __launch_bounds__(256) void conv_chan_dx(ChanArgs g, const T* __restrict__ err, const T* __restrict__ w,
                                                    T* __restrict__ dx) {
    constexpr int EP = DT_X + MAX_KW;
    constexpr int ER = DT_Y + MAX_KH - 1;
    __shared__ T etile[ER * EP];
    __shared__ T taps[64 * MAX_KH * MAX_KW / 4];   // taps of the channels this block handles (up to 16)
    const int x0 = blockIdx.x * DT_X, y0 = blockIdx.y * DT_Y;
    const int c_begin = blockIdx.z * g.cps;
    int c_end = c_begin + g.cps; if (c_end > g.C) c_end = g.C;
    const int ew = DT_X + g.KW - 1, eh = DT_Y + g.KH - 1;
    // error halo: rows y0-(KH-1) .. y0+DT_Y-1, cols x0-(KW-1) .. x0+DT_X-1
    for (int idx = threadIdx.x; idx < eh * ew; idx += 256) {
        const int r = idx / ew, cc = idx % ew;
        const int y = y0 - (g.KH - 1) + r, x = x0 - (g.KW - 1) + cc;
        T v = T(0);
        if (y >= 0 && y < g.OH && x >= 0 && x < g.OW) v = err[(int64_t)y * g.OW + x];
        etile[r * EP + cc] = v;
    }
    const int ntaps = g.KH * g.KW;
    for (int idx = threadIdx.x; idx < (c_end - c_begin) * ntaps; idx += 256) taps[idx] = w[(int64_t)c_begin * ntaps + idx];
    __syncthreads();
    const int lane_x = threadIdx.x & 63, wy = threadIdx.x >> 6;    // 4 row groups of DT_Y/4 rows
    for (int c = c_begin; c < c_end; c++) {
        const T* t = &taps[(c - c_begin) * ntaps];
        T acc[DT_Y / 4];
#pragma unroll
        for (int r = 0; r < DT_Y / 4; r++) acc[r] = T(0);
        for (int ky = 0; ky < g.KH; ky++)
            for (int kx = 0; kx < g.KW; kx++) {
                const T tv = t[ky * g.KW + kx];
#pragma unroll
                for (int r = 0; r < DT_Y / 4; r++) {
                    const int ry = wy * (DT_Y / 4) + r;
                    // err[y-ky][x-kx] -> tile row ry + (KH-1) - ky, col lane_x + (KW-1) - kx
                    acc[r] = __builtin_fma(etile[(ry + g.KH - 1 - ky) * EP + lane_x + g.KW - 1 - kx], tv, acc[r]);
                }
            }
        const int x = x0 + lane_x;
#pragma unroll
        for (int r = 0; r < DT_Y / 4; r++) {
            const int y = y0 + wy * (DT_Y / 4) + r;
            if (y < g.H && x < g.W) dx[((int64_t)c * g.H + y) * g.W + x] = acc[r];
        }
    }
}

// chan_dk: dk[c][ky][kx] = sum_y sum_x in[c][y+ky][x+kx] * err[y][x]; one block per (c, row band),
// every thread accumulates all taps over its share of the band, then a block-wide reduction.
template <typename T>
__global__ __launch_bounds__(256) void conv_chan_dk(ChanArgs g, int bands, int rows_per_band, const T* __restrict__ in,
                                                    const T* __restrict__ err, T* __restrict__ partial) {
    __shared__ T red[4][MAX_KH * MAX_KW];
    const int c = blockIdx.x, band = blockIdx.y;
    const int ya = band * rows_per_band;
    int yb = ya + rows_per_band; if (yb > g.OH) yb = g.OH;
    const T* plane = in + (int64_t)c * g.H * g.W;
    T acc[MAX_KH * MAX_KW];
#pragma unroll
    for (int t = 0; t < MAX_KH * MAX_KW; t++) acc[t] = T(0);
    for (int y = ya; y < yb; y++)
        for (int x = threadIdx.x; x < g.OW; x += 256) {
            const T e = err[(int64_t)y * g.OW + x];
#pragma unroll
            for (int ky = 0; ky < MAX_KH; ky++)
#pragma unroll
                for (int kx = 0; kx < MAX_KW; kx++)
                    if (ky < g.KH && kx < g.KW)
                        acc[ky * MAX_KW + kx] = __builtin_fma(plane[(int64_t)(y + ky) * g.W + x + kx], e, acc[ky * MAX_KW + kx]);
        }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int ky = 0; ky < MAX_KH; ky++)
#pragma unroll
        for (int kx = 0; kx < MAX_KW; kx++)
            if (ky < g.KH && kx < g.KW) {
                T v = acc[ky * MAX_KW + kx];
#pragma unroll
                for (int off = 32; off >= 1; off >>= 1) v += __shfl_down(v, off, 64);
                if (lane == 0) red[wave][ky * MAX_KW + kx] = v;
            }
    __syncthreads();
    if (threadIdx.x < MAX_KH * MAX_KW) {
        const int ky = threadIdx.x / MAX_KW, kx = threadIdx.x % MAX_KW;
        if (ky < g.KH && kx < g.KW) {
            T s = (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
            partial[((int64_t)band * g.C + c) * (g.KH * g.KW) + ky * g.KW + kx] = s;
        }
    }
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

template <typename T>
static int conv_typed(Device* dev, int d, int rank, nk_buf drn, const Cfg& c0, nk_buf a, const Cfg& c1, nk_buf b,
                      const Cfg& c2, int64_t n) {
    T* out = (T*)drn;
    const T* s1 = (const T*)a;
    const T* s2 = (const T*)b;
    const bool dense = dense_rm(c0, rank) && dense_rm(c1, rank) && dense_rm(c2, rank);
    if (dense && rank == 3 && sizeof(T) == 4) {
        if (d < 0 && c0.shape[0] == 1 && c1.shape[0] == c2.shape[0] && c1.shape[0] > 1) {
            // which operand is the big one?
            const bool a_big = c1.shape[1] >= c2.shape[1] && c1.shape[2] >= c2.shape[2];
            const bool b_big = c2.shape[1] >= c1.shape[1] && c2.shape[2] >= c1.shape[2];
            if (a_big || b_big) {
                const Cfg& big = a_big ? c1 : c2;
                const Cfg& small = a_big ? c2 : c1;
                if (small.shape[1] <= MAX_KH && small.shape[2] <= MAX_KW) {
                    ChanArgs g{};
                    g.C = big.shape[0]; g.H = big.shape[1]; g.W = big.shape[2];
                    g.KH = small.shape[1]; g.KW = small.shape[2];
                    g.OH = g.H - g.KH + 1; g.OW = g.W - g.KW + 1;
                    const int tiles = ((g.OW + FT_X - 1) / FT_X) * ((g.OH + FT_Y - 1) / FT_Y);
                    int splits = (dev->props.multiProcessorCount * 2 + tiles - 1) / tiles;
                    if (splits > (g.C + 3) / 4) splits = (g.C + 3) / 4;
                    if (splits < 1) splits = 1;
                    g.cps = (g.C + splits - 1) / splits;
                    splits = (g.C + g.cps - 1) / g.cps;
                    g.splits = splits;
                    void* ws = nullptr;
                    if (int e = workspace(dev, (uint64_t)splits * g.OH * g.OW * sizeof(T), &ws)) return e;
                    dim3 grid((g.OW + FT_X - 1) / FT_X, (g.OH + FT_Y - 1) / FT_Y, splits);
                    set_path("chan_fwd");
                    const T* bigp = a_big ? s1 : s2;
                    const T* smallp = a_big ? s2 : s1;
                    if (g.KH == 5 && g.KW == 5)
                        hipLaunchKernelGGL((conv_chan_fwd<T, 5, 5>), grid, dim3(256), 0, dev->stream, g, bigp, smallp, (T*)ws);
                    else if (g.KH == 3 && g.KW == 3)
                        hipLaunchKernelGGL((conv_chan_fwd<T, 3, 3>), grid, dim3(256), 0, dev->stream, g, bigp, smallp, (T*)ws);
                    else
                        hipLaunchKernelGGL((conv_chan_fwd<T, 0, 0>), grid, dim3(256), 0, dev->stream, g, bigp, smallp, (T*)ws);
                    NK_HIP(hipGetLastError());
                    const int on = g.OH * g.OW;
                    hipLaunchKernelGGL(conv_chan_fwd_reduce<T>, dim3((on + 255) / 256), dim3(256), 0, dev->stream, splits, on, (const T*)ws, out);
                    NK_HIP(hipGetLastError());
                    return NK_OK;
                }
            }
        }
        if (d >= 0 && c2.shape[0] == 1 && c0.shape[0] == c1.shape[0] && c0.shape[0] > 1) {
            // src2 = error [1,OH,OW]
            const int OH = c2.shape[1], OW = c2.shape[2];
            // dx: drain [C,H,W] bigger than src1 = taps [C,KH,KW] with H = OH + KH - 1
            if (c0.shape[1] >= c1.shape[1] && c0.shape[2] >= c1.shape[2] && c1.shape[1] <= MAX_KH && c1.shape[2] <= MAX_KW &&
                c0.shape[1] == OH + c1.shape[1] - 1 && c0.shape[2] == OW + c1.shape[2] - 1 &&
                (c0.shape[1] > c1.shape[1] || c1.shape[1] == 1) && (c0.shape[2] > c1.shape[2] || c1.shape[2] == 1)) {
                ChanArgs g{};
                g.C = c0.shape[0]; g.H = c0.shape[1]; g.W = c0.shape[2];
                g.KH = c1.shape[1]; g.KW = c1.shape[2]; g.OH = OH; g.OW = OW;
                g.cps = 4;
                g.splits = (g.C + g.cps - 1) / g.cps;
                dim3 grid((g.W + DT_X - 1) / DT_X, (g.H + DT_Y - 1) / DT_Y, g.splits);
                set_path("chan_dx");
                hipLaunchKernelGGL(conv_chan_dx<T>, grid, dim3(256), 0, dev->stream, g, s2, s1, out);
                NK_HIP(hipGetLastError());
                return NK_OK;
            }
            // dk: drain [C,KH,KW] smaller than src1 = input [C,H,W]
            if (c0.shape[1] <= MAX_KH && c0.shape[2] <= MAX_KW && c1.shape[1] == OH + c0.shape[1] - 1 &&
                c1.shape[2] == OW + c0.shape[2] - 1 && c0.shape[1] < c1.shape[1] && c0.shape[2] < c1.shape[2]) {
                ChanArgs g{};
                g.C = c0.shape[0]; g.H = c1.shape[1]; g.W = c1.shape[2];
                g.KH = c0.shape[1]; g.KW = c0.shape[2]; g.OH = OH; g.OW = OW;
                int bands = (dev->props.multiProcessorCount * 4 + g.C - 1) / g.C;
                if (bands > OH) bands = OH;
                if (bands < 1) bands = 1;
                const int rpb = (OH + bands - 1) / bands;
                bands = (OH + rpb - 1) / rpb;
                const int ntaps = g.KH * g.KW;
                void* ws = nullptr;
                if (int e = workspace(dev, (uint64_t)bands * g.C * ntaps * sizeof(T), &ws)) return e;
                set_path("chan_dk");
                hipLaunchKernelGGL(conv_chan_dk<T>, dim3(g.C, bands), dim3(256), 0, dev->stream, g, bands, rpb, s1, s2, (T*)ws);
                NK_HIP(hipGetLastError());
                const int on = g.C * ntaps;
                hipLaunchKernelGGL(conv_chan_fwd_reduce<T>, dim3((on + 255) / 256), dim3(256), 0, dev->stream, bands, on, (const T*)ws, out);
                NK_HIP(hipGetLastError());
                return NK_OK;
            }
        }
    }
    ConvArgs A{};
    A.rank = rank; A.n = (unsigned)n; A.c0 = c0; A.c1 = c1; A.c2 = c2;
    unsigned blocks = (unsigned)((n + 255) / 256);
    if (blocks > 65536) blocks = 65536;
    set_path(d < 0 ? "literal_fwd" : "literal_bwd");
    if (d < 0) hipLaunchKernelGGL(conv_fwd_literal<T>, dim3(blocks), dim3(256), 0, dev->stream, A, out, s1, s2);
    else       hipLaunchKernelGGL(conv_bwd_literal<T>, dim3(blocks), dim3(256), 0, dev->stream, A, out, s1, s2);
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
    return dtype == NK_F32 ? conv_typed<float>(dev, d, rank, drn, c0, a, c1, b, c2, n)
                           : conv_typed<double>(dev, d, rank, drn, c0, a, c1, b, c2, n);
}
