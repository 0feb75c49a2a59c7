// nk_scalarization_int: drain = src op value for the integer element types.
//
// The reference generates its scalarization kernel for "int", "long", "short" and "char" beside the two float
// types (J/backend/main/implementations/broadcast/CLScalarBroadcast.java:40-58).  The arithmetic here is the CPU
// device's (CPUScalarBroadcast.java:83-190 with the functions of CPUScalarBroadcastAddition / Subtraction /
// Multiplication / Division / Modulo / Identity and CPUScalaBroadcastPower, and the defaults of
// fun/api/CPUBiFun.java:9-27):
//   int, long    + - * wrap; / and % truncate like Java's (MIN / -1 = MIN, x % -1 = 0; a zero divisor is an
//                ArithmeticException there and an argument error here); power and every derivative that needs
//                it go through double and Math.round.
//   short, byte  have no overloads of their own: every function is evaluated in double and narrowed with
//                (short) Math.round(..) / (byte) Math.round(..), so 7 / 2 is 4 and x / 0 is -1.
// Math.round(double) is floor(x + 1/2) evaluated exactly, saturates at the ends of long and maps NaN to 0.
//
// Two kernels: dense operands with the same layout move 16 bytes per lane; everything else goes through the
// descriptors element by element.  The operator is selected once per thread, outside the element loop.
#include "nk_internal.h"
#include "nk_scalar.h"
#include <type_traits>

namespace nk {

__device__ inline int64_t java_round(double x) {
    if (x != x) return 0;
    if (x >= 9223372036854775807.0) return INT64_MAX;
    if (x <= -9223372036854775808.0) return INT64_MIN;
    const double f = floor(x);
    int64_t r = (int64_t)f;
    if (x - f >= 0.5) r += 1;                      // x - floor(x) is exact
    return r;
}

// mode = op * 3 + (d + 1): d = -1 the function, 0 / 1 its derivative by the element / by the value
template <typename I, int MODE>
__device__ inline I int_apply(I a, I b) {
    constexpr int OP = MODE / 3, D = MODE % 3 - 1;
    using U = std::make_unsigned_t<I>;
    constexpr bool WIDE = sizeof(I) >= 4;          // int and long have integer overloads, short and byte do not
    if constexpr (OP == NK_OP_IDY) return b;
    if constexpr (WIDE) {
        if constexpr (OP == NK_OP_ADD) return D < 0 ? (I)((U)a + (U)b) : (I)1;
        if constexpr (OP == NK_OP_SUB) return D < 0 ? (I)((U)a - (U)b) : (D == 0 ? (I)1 : (I)-1);
        if constexpr (OP == NK_OP_MUL) return D < 0 ? (I)((U)a * (U)b) : (D == 0 ? b : a);
        if constexpr (OP == NK_OP_DIV || OP == NK_OP_MOD) {
            if constexpr (D < 0) {                 // b != 0 is checked on the host
                if (b == (I)-1) return OP == NK_OP_DIV ? (I)((U)0 - (U)a) : (I)0;
                return OP == NK_OP_DIV ? (I)(a / b) : (I)(a % b);
            }
            if constexpr (D == 0) return (I)java_round(1.0 / (double)b);
            const I neg = (I)((U)0 - (U)a);        // -a in the element type, then -a / Math.pow(b, 2)
            return (I)java_round((double)neg / ((double)b * (double)b));
        }
        if constexpr (OP == NK_OP_POW) {
            if constexpr (D < 0) return (I)java_round(pow_ref((double)a, (double)b));
            if constexpr (D == 0) return (I)java_round((double)b * pow_ref((double)a, (double)(I)((U)b - (U)1)));
            return (I)java_round(pow_ref((double)a, (double)b) * log((double)a));
        }
    } else {
        const double x = (double)a, y = (double)b;
        double r = 0.0;
        if constexpr (OP == NK_OP_ADD) r = D < 0 ? x + y : 1.0;
        if constexpr (OP == NK_OP_SUB) r = D < 0 ? x - y : (D == 0 ? 1.0 : -1.0);
        if constexpr (OP == NK_OP_MUL) r = D < 0 ? x * y : (D == 0 ? y : x);
        if constexpr (OP == NK_OP_DIV || OP == NK_OP_MOD) {
            if constexpr (D < 0) r = OP == NK_OP_DIV ? x / y : fmod(x, y);
            if constexpr (D == 0) r = 1.0 / y;
            if constexpr (D == 1) r = -(x / (y * y));
        }
        if constexpr (OP == NK_OP_POW) {
            if constexpr (D < 0) r = pow_ref(x, y);
            if constexpr (D == 0) r = y * pow_ref(x, y - 1.0);
            if constexpr (D == 1) r = pow_ref(x, y) * log(x);
        }
        return (I)java_round(r);                   // narrowing keeps the low bits, as Java's casts do
    }
    return (I)0;
}

template <typename Body>
__device__ inline void for_mode(int mode, Body body) {
    switch (mode) {
#define NK_MODE(M) case M: body(std::integral_constant<int, M>{}); break;
        NK_MODE(0) NK_MODE(1) NK_MODE(2) NK_MODE(3) NK_MODE(4) NK_MODE(5) NK_MODE(6) NK_MODE(7) NK_MODE(8) NK_MODE(9)
        NK_MODE(10) NK_MODE(11) NK_MODE(12) NK_MODE(13) NK_MODE(14) NK_MODE(15) NK_MODE(16) NK_MODE(17) NK_MODE(18)
        NK_MODE(19) NK_MODE(20)
#undef NK_MODE
        default: break;
    }
}

// dense, same layout: n_vec pieces of 16 bytes, then a tail of single elements
template <typename I>
__global__ __launch_bounds__(256) void int_scalar_flat(int mode, I value, int64_t n, I* __restrict__ drn, const I* __restrict__ src) {
    constexpr int VEC = 16 / sizeof(I);
    typedef I Vec __attribute__((ext_vector_type(VEC)));
    const int64_t n_vec = n / VEC;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    const int64_t first = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    for_mode(mode, [&](auto M) {
        constexpr int MODE = decltype(M)::value;
        for (int64_t p = first; p < n_vec; p += step) {
            const Vec v = __builtin_nontemporal_load((const Vec*)src + p);
            Vec r;
#pragma unroll
            for (int e = 0; e < VEC; e++) r[e] = int_apply<I, MODE>(v[e], value);
            ((Vec*)drn)[p] = r;
        }
        for (int64_t i = n_vec * VEC + first; i < n; i += step) drn[i] = int_apply<I, MODE>(src[i], value);
    });
}

// any pair of views: flat index -> position through each operand's own descriptor
template <typename I>
__global__ __launch_bounds__(256) void int_scalar_indexed(int mode, I value, int rank, unsigned n, Cfg c0, Cfg c1, I* __restrict__ drn,
                                                          const I* __restrict__ src) {
    const unsigned step = gridDim.x * blockDim.x;
    const unsigned first = blockIdx.x * blockDim.x + threadIdx.x;
    for_mode(mode, [&](auto M) {
        constexpr int MODE = decltype(M)::value;
        for (unsigned i = first; i < n; i += step)
            drn[phys_of_flat(c0, rank, (int)i)] = int_apply<I, MODE>(src[phys_of_flat(c1, rank, (int)i)], value);
    });
}

static bool dense_row_major(const Cfg& c, int rank) {
    int64_t stride = 1;
    for (int k = rank - 1; k >= 0; k--) {
        if (c.spread[k] != 1 || c.offset[k] != 0 || c.strides[k] != stride || c.imap[k] != stride) return false;
        stride *= c.shape[k];
    }
    return true;
}

template <typename I>
static int int_scalar_typed(Device* dev, int mode, int64_t value, int rank, nk_buf drn, const Cfg& c0, nk_buf src, const Cfg& c1, int64_t n) {
    const I v = (I)value;                          // Number.intValue() / shortValue() / ...: the low bits
    const int cus = dev->props.multiProcessorCount;
    bool same = true;
    for (int k = 0; k < rank; k++) same = same && c0.shape[k] == c1.shape[k];
    if (same && dense_row_major(c0, rank) && dense_row_major(c1, rank) && drn % 16 == 0 && src % 16 == 0) {
        constexpr int VEC = 16 / sizeof(I);
        int64_t blocks = (n / VEC + 255) / 256;
        if (blocks < 1) blocks = 1;
        if (blocks > (int64_t)cus * 32) blocks = (int64_t)cus * 32;
        set_path("int_flat");
        hipLaunchKernelGGL(int_scalar_flat<I>, dim3((unsigned)blocks), dim3(256), 0, dev->stream, mode, v, n, (I*)drn, (const I*)src);
    } else {
        int64_t blocks = (n + 255) / 256;
        if (blocks > (int64_t)cus * 32) blocks = (int64_t)cus * 32;
        set_path("int_indexed");
        hipLaunchKernelGGL(int_scalar_indexed<I>, dim3((unsigned)blocks), dim3(256), 0, dev->stream, mode, v, rank, (unsigned)n, c0, c1, (I*)drn, (const I*)src);
    }
    NK_HIP(hipGetLastError());
    return NK_OK;
}

}  // namespace nk

using namespace nk;

extern "C" int nk_scalarization_int(nk_dev h, int op_id, int d, int dtype, int rank, nk_buf drn, const int32_t* drn_cfg,
                                    nk_buf src, const int32_t* src_cfg, int64_t value, int64_t n) {
    NK_DEVICE(dev, h);
    NK_REQUIRE(dtype == NK_I32 || dtype == NK_I64 || dtype == NK_I16 || dtype == NK_I8, "nk_scalarization_int: dtype %d is not an integer type", dtype);
    NK_REQUIRE(op_id >= NK_OP_ADD && op_id <= NK_OP_IDY, "nk_scalarization_int: unknown operator %d", op_id);
    NK_REQUIRE(d >= -1 && d <= 1, "nk_scalarization_int: derivative index %d outside [-1, 1]", d);
    if (int e = check_cfg("nk_scalarization_int(drain)", drn_cfg, rank)) return e;
    if (int e = check_cfg("nk_scalarization_int(src)", src_cfg, rank)) return e;
    int64_t size = 1, src_size = 1;
    for (int k = 0; k < rank; k++) { size *= drn_cfg[k]; src_size *= src_cfg[k]; }
    NK_REQUIRE(n == size && n == src_size && size < ((int64_t)1 << 31),
               "nk_scalarization_int: n = %lld, the drain holds %lld and the source %lld elements", (long long)n, (long long)size, (long long)src_size);
    const int eb = dtype == NK_I64 ? 8 : dtype == NK_I32 ? 4 : dtype == NK_I16 ? 2 : 1;
    NK_REQUIRE(drn % eb == 0 && src % eb == 0, "nk_scalarization_int: operands must be aligned to their element size");
    if (int e = check_extent(dev, "nk_scalarization_int(drain)", drn, drn_cfg, rank, eb)) return e;
    if (int e = check_extent(dev, "nk_scalarization_int(src)", src, src_cfg, rank, eb)) return e;
    if (d < 0 && (op_id == NK_OP_DIV || op_id == NK_OP_MOD) && (dtype == NK_I32 || dtype == NK_I64)) {
        const int64_t narrowed = dtype == NK_I32 ? (int64_t)(int32_t)value : value;
        NK_REQUIRE(narrowed != 0, "nk_scalarization_int: / by zero");        // java.lang.ArithmeticException on the CPU device
    }
    Cfg c0, c1;
    load_cfg(c0, drn_cfg, rank); load_cfg(c1, src_cfg, rank);
    tame_unravel(c0, rank, n); tame_unravel(c1, rank, n);
    const int mode = op_id * 3 + (d + 1);
    switch (dtype) {
        case NK_I32: return int_scalar_typed<int32_t>(dev, mode, value, rank, drn, c0, src, c1, n);
        case NK_I64: return int_scalar_typed<int64_t>(dev, mode, value, rank, drn, c0, src, c1, n);
        case NK_I16: return int_scalar_typed<int16_t>(dev, mode, value, rank, drn, c0, src, c1, n);
        default:     return int_scalar_typed<int8_t>(dev, mode, value, rank, drn, c0, src, c1, n);
    }
}
