/*
 * neureka_cpu_oracle.c — TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C restatement of the algorithms of Neureka's `CPU` device for the HipDevice hot path.  It is
 * the checker the HIP kernels are compared against; only tests, the smoke check and the CPU-baseline
 * leg of the benchmark may load it.  The shipped library never calls into this file.
 *
 * The reference is Java and no JVM exists where this is built, so nothing here was checked by running
 * the reference.  What pins each function (see tests/test_oracle_*.py):
 *   index maths            the 20 descriptor rows of NDConfiguration_Spec, slice/permute strings of
 *                          Tensor_Slice_Permute_Spec, brute force against numpy strides
 *   seeded generator       the enforced sums of Calculus_Stress_Test ("Tempeh", "Seitan" vectors)
 *   activations            the same sums and the silu/gelu/selu/gatu/gasu value+derivative vectors;
 *                          every function also against closed forms evaluated by numpy in float64
 *   broadcast fwd/bwd      literal vectors of Tensor_Operation_Spec / Calculus_Stress_Test; numpy
 *                          broadcasting (forward) and numpy sums (backward)
 *   convolution fwd/bwd    literal vectors of Tensor_Convolution_Spec, CrossDeviceSystemTest;
 *                          scipy.signal.correlate; the state machines against the closed forms
 *   matmul                 hash known-answers of InternalMatMulTest; numpy matmul on integer data
 *   power                  the table of special cases in the Javadoc of Math.pow (where C's pow differs the
 *                          reference's answer is kept)
 *   reductions             the literal results of Tensor_Stats_Spec / Tensor_Dot_Product_Spec; the tree against
 *                          its own definition and numpy on integer data
 *   integer scalar         the enforced Integer / Long rows of Tensor_Operation_Spec, the Java language rules
 *   broadcast              (wrapping, truncating division, Math.round) against exact integer arithmetic
 *   JVMExecutor split      leaf-count / coverage properties (no golden vector exists: "parity
 *                          unpinned" beyond those properties; it only affects baseline timing)
 *
 * Citations: J/ = src/main/java/neureka/ of the reference.
 *
 * Build: gcc -O2 -fPIC -shared -ffp-contract=off -fno-fast-math (see Makefile): + - * / must stay single
 * IEEE operations, exactly as the JVM evaluates them.
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* java.lang.Math.pow where it differs from C99's pow: a NaN exponent gives NaN whatever the base (C: pow(1, NaN) = 1)
 * and a base of magnitude 1 with an infinite exponent gives NaN (C: 1).  Every other special case of the Javadoc
 * table (x^0 = 1 also for NaN, negative base with a non-integer exponent = NaN, signed zeros and infinities) is C99's
 * Annex F behaviour.  Exported for the tests that check the table. */
double orc_java_pow(double a, double b) {
    if (b == 0.0) return 1.0;
    if (b != b) return (double)NAN;
    if (fabs(a) == 1.0 && isinf(b)) return (double)NAN;
    return pow(a, b);
}


#define ORC_MAX_RANK 8

/* ------------------------------------------------------------------------------------------------
 * View descriptors: int32[5*rank] = shape | strides | indicesMap | offset | spread
 * (NDConfiguration.asInlineArray, J/ndim/config/NDConfiguration.java:335-345).
 */
typedef struct {
    int rank;
    const int32_t *shape, *strides, *imap, *offset, *spread;
} view_t;

static view_t view_of(const int32_t* cfg, int rank) {
    view_t v = {rank, cfg, cfg + rank, cfg + 2 * rank, cfg + 3 * rank, cfg + 4 * rank};
    return v;
}

/* indicesOfIndex: J/ndim/config/types/sliced/SlicedNDConfiguration.java:94-102.
 * A virtual descriptor (all-zero tables) maps everything to 0: VirtualNDConfiguration.java:34-64. */
static void indices_of_index(const view_t* v, int index, int* indices) {
    for (int i = 0; i < v->rank; i++) {
        indices[i] = 0;
        if (v->imap[i] != 0) {
            indices[i] += index / v->imap[i];
            index %= v->imap[i];
        }
    }
}

/* indexOfIndices: SlicedNDConfiguration.java:104-111 (Java int arithmetic: wraps) */
static int index_of_indices(const view_t* v, const int* indices) {
    int32_t index = 0;
    for (int i = 0; i < v->rank; i++)
        index += (int32_t)((uint32_t)((int32_t)((uint32_t)indices[i] * (uint32_t)v->spread[i]) + v->offset[i]) * (uint32_t)v->strides[i]);
    return index;
}

int orc_index_of_index(const int32_t* cfg, int rank, int index) {
    view_t v = view_of(cfg, rank);
    int idx[ORC_MAX_RANK];
    indices_of_index(&v, index, idx);
    return index_of_indices(&v, idx);
}

/* NDConfiguration.Utility.increment (NDConfiguration.java:436-451): last axis fastest */
static void increment(int* indices, const int32_t* shape, int rank) {
    int i = rank - 1;
    while (i >= 0 && i < rank) {
        if (indices[i] < shape[i]) {
            indices[i]++;
            if (indices[i] == shape[i]) { indices[i] = 0; i--; }
            else i = -1;
        } else i--;
    }
}

static int view_size(const view_t* v) {
    int s = 1;
    for (int i = 0; i < v->rank; i++) s *= v->shape[i];
    return s;
}

/* ------------------------------------------------------------------------------------------------
 * Scalar functions, J/backend/main/implementations/fun/Scalar*.java.
 * f64: the `double invoke(double)` lambdas.  f32: the `float invoke(float)` overrides where a class
 * has one, else CPUFun's default `(float) invoke((double) x)` (fun/api/CPUFun.java:7-9).
 */
enum {
    FUN_ABS = 0, FUN_COS, FUN_GASU, FUN_GATU, FUN_GAUS, FUN_FAST_GAUS, FUN_GELU, FUN_IDY, FUN_LN, FUN_QUAD,
    FUN_RELU, FUN_SELU, FUN_SIG, FUN_SILU, FUN_SIN, FUN_SOFTPLUS, FUN_SOFTSIGN, FUN_TANH, FUN_FAST_TANH,
    FUN_EXP, FUN_LOG10, FUN_SQRT, FUN_CBRT, FUN_COUNT
};

static const double SELU_ALPHA = 1.6732632423543772848170429916717;
static const double SELU_SCALE = 1.0507009873554804934193349852946;

/* FunUtil.invSqrt, fun/FunUtil.java:5-27 */
static double inv_sqrt_f64(double x) {
    double xhalf = 0.5 * x;
    int64_t i;
    memcpy(&i, &x, 8);
    i = 0x5fe6ec85e7de30daLL - (i >> 1);
    memcpy(&x, &i, 8);
    x *= (1.5 - xhalf * x * x);
    x *= (1.5 - xhalf * x * x);
    x *= (1.5 - xhalf * x * x);
    x *= (1.5 - xhalf * x * x);
    return x;
}
static float inv_sqrt_f32(float x) {
    float xhalf = 0.5f * x;
    int32_t i;
    memcpy(&i, &x, 4);
    i = 0x5f3759df - (i >> 1);
    memcpy(&x, &i, 4);
    x *= (1.5f - xhalf * x * x);
    x *= (1.5f - xhalf * x * x);
    return x;
}

static double sig64(double x) { return 1.0 / (1.0 + exp(-x)); }                       /* ScalarSigmoid.java:38 */
static double tanh64(double x) { return 2 / (1 + exp(-x * 2)) - 1; }                  /* ScalarTanh.java:37 */
static float tanh32(float x) { return (float)(2 / (1 + exp((double)(-x * 2))) - 1); } /* ScalarTanh.java:38, -x*2 is a float product */
static double softsign64(double x) { return x / (1.0 + fabs(x)); }                    /* ScalarSoftsign.java */
static float softsign32(float x) { return x / (1.0f + fabsf(x)); }
static double selu64(double x) {                                                      /* ScalarSeLU.java */
    if (x > 0) return SELU_SCALE * x;
    else if (x <= 0) return SELU_SCALE * SELU_ALPHA * (exp(x) - 1);
    else return (double)NAN;
}

double orc_fun_f64(int id, int derive, double x) {
    if (!derive) switch (id) {
        case FUN_ABS: return fabs(x);
        case FUN_COS: return cos(x);
        case FUN_GASU: return softsign64(x * x * x);
        case FUN_GATU: return tanh64(x * x * x);
        case FUN_GAUS: return exp(-(x * x));
        case FUN_FAST_GAUS: return 1 / (1 + x * x);
        case FUN_GELU: return x * sig64(x * 1.702);
        case FUN_IDY: return x;
        case FUN_LN: return log(x);
        case FUN_QUAD: return x * x;
        case FUN_RELU: return (x >= 0 ? x : x * .01);
        case FUN_SELU: return selu64(x);
        case FUN_SIG: return sig64(x);
        case FUN_SILU: return x * sig64(x);
        case FUN_SIN: return sin(x);
        case FUN_SOFTPLUS: return log(1.0 + exp(x));
        case FUN_SOFTSIGN: return softsign64(x);
        case FUN_TANH: return tanh64(x);
        case FUN_FAST_TANH: return x * inv_sqrt_f64(1.0 + x * x);
        case FUN_EXP: return exp(x);
        case FUN_LOG10: return log10(x);
        case FUN_SQRT: return sqrt(x);
        case FUN_CBRT: return cbrt(x);
    } else switch (id) {
        case FUN_ABS: return (x < 0.0 ? -1.0 : 1.0);
        case FUN_COS: return -sin(x);
        case FUN_GASU: { double x2 = x * x, x6 = x2 * x2 * x2; return 3.0 * x2 / (2.0 * x2 * fabs(x) + x6 + 1.0); }
        case FUN_GATU: { double x2 = x * x, x3 = x2 * x, temp = 3 * x2, t2 = orc_java_pow(tanh64(x3), 2); return -temp * t2 + temp; }
        case FUN_GAUS: return -2 * x * exp(-(x * x));
        case FUN_FAST_GAUS: { double x2 = x * x; return -2 * x / (x2 * x2 + 2 * x2 + 1); }
        case FUN_GELU: { double s = sig64(x * 1.702), ds = s * (1.0 - s); return s + ds * x * 1.702; }
        case FUN_IDY: return 1;
        case FUN_LN: return 1.0 / x;
        case FUN_QUAD: return 2 * x;
        case FUN_RELU: return (x >= 0 ? 1 : .01);
        case FUN_SELU: if (x > 0) return SELU_SCALE; else if (x <= 0) return SELU_SCALE * SELU_ALPHA * exp(x); else return (double)NAN;
        case FUN_SIG: { double s = sig64(x); return s * (1 - s); }
        case FUN_SILU: { double s = sig64(x); return s + (x * s * (1.0 - s)); }
        case FUN_SIN: return cos(x);
        case FUN_SOFTPLUS: return 1.0 / (1.0 + exp(-x));
        case FUN_SOFTSIGN: return 1.0 / (2.0 * fabs(x) + x * x + 1.0);
        case FUN_TANH: return 1 - orc_java_pow(tanh64(x), 2);
        case FUN_FAST_TANH: { double t1 = x * x, t2 = sqrt(1 + t1); return 1 / (t1 * t2 + t2); }
        case FUN_EXP: return exp(x);
        case FUN_LOG10: return 1 / (x * log(10));
        case FUN_SQRT: return 0.5 * inv_sqrt_f64(x);
        case FUN_CBRT: return 1 / (3 * orc_java_pow(x, 2.0 / 3.0));
    }
    return (double)NAN;
}

float orc_fun_f32(int id, int derive, float x) {
    if (!derive) switch (id) {
        case FUN_ABS: return fabsf(x);
        case FUN_GASU: return softsign32(x * x * x);
        case FUN_GATU: return tanh32(x * x * x);
        case FUN_FAST_GAUS: return 1 / (1 + x * x);
        case FUN_IDY: return x;
        case FUN_QUAD: return x * x;
        case FUN_RELU: return (x >= 0 ? x : x * .01f);
        case FUN_SOFTSIGN: return softsign32(x);
        case FUN_TANH: return tanh32(x);
        case FUN_FAST_TANH: return x * inv_sqrt_f32(1.0f + x * x);
        default: return (float)orc_fun_f64(id, 0, (double)x);     /* CPUFun default and the (float) Math.f(x) overrides */
    } else switch (id) {
        case FUN_ABS: return (x < 0.0f ? -1.0f : 1.0f);
        case FUN_CBRT: return 1 / (3 * (float)orc_java_pow((double)x, (double)(2.0f / 3.0f)));
        case FUN_EXP: return (float)exp((double)x);
        case FUN_GASU: { float x2 = x * x, x6 = x2 * x2 * x2; return 3.0f * x2 / (2.0f * x2 * fabsf(x) + x6 + 1.0f); }
        case FUN_GATU: { float x2 = x * x, x3 = x2 * x, temp = 3 * x2, t2 = (float)orc_java_pow((double)tanh32(x3), 2); return -temp * t2 + temp; }
        case FUN_FAST_GAUS: { float x2 = x * x; return -2 * x / (x2 * x2 + 2 * x2 + 1); }
        case FUN_GELU: { float s = (float)sig64((double)x * 1.702), ds = s * (1.0f - s); return s + ds * x * 1.702f; }
        case FUN_IDY: return 1;
        case FUN_LN: return 1.0f / x;
        case FUN_LOG10: return 1 / (x * (float)log(10));
        case FUN_QUAD: return 2 * x;
        case FUN_RELU: return (x >= 0 ? 1.0f : .01f);
        case FUN_SELU: if (x > 0) return (float)SELU_SCALE; else if (x <= 0) return (float)(SELU_SCALE * SELU_ALPHA * exp((double)x)); else return NAN;
        case FUN_SIG: { float s = (float)sig64((double)x); return s * (1 - s); }
        case FUN_SILU: { float s = (float)sig64((double)x); return s + (x * s * (1.0f - s)); }
        case FUN_SOFTSIGN: return 1.0f / (2.0f * fabsf(x) + x * x + 1.0f);
        case FUN_SQRT: return 0.5f * inv_sqrt_f32(x);
        case FUN_TANH: return (float)(1 - orc_java_pow((double)tanh32(x), 2));
        case FUN_FAST_TANH: { float t1 = x * x, t2 = (float)sqrt((double)(1 + t1)); return 1 / (t1 * t2 + t2); }
        default: return (float)orc_fun_f64(id, 1, (double)x);
    }
}

/* binary operators.  family: 0 = same-shape elementwise (CPUBiElementWise*.java), 1 = scalar broadcast
 * (CPUScalarBroadcast*.java, CPUScalaBroadcastPower.java), 2 = broadcast (CPUBroadcast*.java).
 * d < 0: the operator; d = 0/1: _getDeriveAt0/_getDeriveAt1 of that family. */
enum { OP_ADD = 0, OP_SUB, OP_MUL, OP_DIV, OP_MOD, OP_POW, OP_IDY };


double orc_bin_f64(int family, int op, int d, double a, double b) {
    if (d < 0) switch (op) {
        case OP_ADD: return a + b;
        case OP_SUB: return a - b;
        case OP_MUL: return a * b;
        case OP_DIV: return a / b;
        case OP_MOD: return fmod(a, b);           /* Java % on doubles */
        case OP_POW: return orc_java_pow(a, b);
        case OP_IDY: return b;
    }
    if (family == 2) switch (op) {
        case OP_ADD: return a + b;
        case OP_SUB: return d == 0 ? a + b : a - b;
        case OP_MUL: return d == 0 ? b : a;
        case OP_DIV: case OP_MOD: return d == 0 ? 1 / b : -(a / orc_java_pow(b, 2));
        case OP_POW: return d == 0 ? a * orc_java_pow(a, b - 1) : orc_java_pow(a, b) * log(a);
    }
    switch (op) {
        case OP_ADD: return 1;
        case OP_SUB: return d == 0 ? 1 : -1;
        case OP_MUL: return d == 0 ? b : a;
        case OP_DIV: case OP_MOD: return d == 0 ? 1.0 / b : -a / orc_java_pow(b, 2);
        case OP_POW: return d == 0 ? b * orc_java_pow(a, b - 1) : orc_java_pow(a, b) * log(a);
        case OP_IDY: return b;   /* CPUScalarBroadcastIdentity.java:25-33: _getDeriveAt0/1 return _getFun() */
    }
    return (double)NAN;
}

float orc_bin_f32(int family, int op, int d, float a, float b) {
    if (d < 0) switch (op) {
        case OP_ADD: return a + b;
        case OP_SUB: return a - b;
        case OP_MUL: return a * b;
        case OP_DIV: return a / b;
        case OP_MOD: return fmodf(a, b);
        case OP_POW: return (float)orc_java_pow((double)a, (double)b);
        case OP_IDY: return b;
    }
    if (family == 2) switch (op) {
        case OP_ADD: return a + b;
        case OP_SUB: return d == 0 ? a + b : a - b;
        case OP_MUL: return d == 0 ? b : a;
        case OP_DIV: case OP_MOD: return d == 0 ? 1 / b : (float)-((double)a / orc_java_pow((double)b, 2));
        case OP_POW: return d == 0 ? (float)((double)a * orc_java_pow((double)a, (double)(b - 1))) : (float)(orc_java_pow((double)a, (double)b) * log((double)a));
    }
    switch (op) {
        case OP_ADD: return 1;
        case OP_SUB: return d == 0 ? 1 : -1;
        case OP_MUL: return d == 0 ? b : a;
        case OP_DIV: case OP_MOD: return d == 0 ? 1.0f / b : (float)-((double)a / orc_java_pow((double)b, 2));
        case OP_POW: return d == 0 ? (float)((double)b * orc_java_pow((double)a, (double)(b - 1))) : (float)(orc_java_pow((double)a, (double)b) * log((double)a));
        case OP_IDY: return b;   /* CPUScalarBroadcastIdentity.java:25-33: _getDeriveAt0/1 return _getFun() */
    }
    return NAN;
}

/* ------------------------------------------------------------------------------------------------
 * Range workloads.  Every kernel below is a `(start, end)` workload over the drain's flat index, as the
 * reference hands them to CPU.JVMExecutor.threaded (J/devices/host/CPU.java:743-797).
 */

/* CPUElementwiseFunction._workloadFor, J/backend/main/implementations/elementwise/CPUElementwiseFunction.java:96-117:
 * both iterators start at the DRAIN's nd-index of `start` and advance in row-major order. */
void orc_activation(int fun_id, int d, int is_f64, int rank, void* drn, const int32_t* drn_cfg, const void* src,
                    const int32_t* src_cfg, int start, int end) {
    view_t v0 = view_of(drn_cfg, rank), v1 = view_of(src_cfg, rank);
    int i0[ORC_MAX_RANK], i1[ORC_MAX_RANK];
    indices_of_index(&v0, start, i0);
    memcpy(i1, i0, sizeof i0);
    for (int i = start; i < end; i++) {
        if (is_f64) ((double*)drn)[index_of_indices(&v0, i0)] = orc_fun_f64(fun_id, d >= 0, ((const double*)src)[index_of_indices(&v1, i1)]);
        else ((float*)drn)[index_of_indices(&v0, i0)] = orc_fun_f32(fun_id, d >= 0, ((const float*)src)[index_of_indices(&v1, i1)]);
        increment(i0, v0.shape, rank);
        increment(i1, v1.shape, rank);
    }
}

/* CPUBiElementWise._newWorkloadF32/F64, elementwise/CPUBiElementWise.java:99-142: every operand
 * unravels `start` with its OWN indicesMap, then all advance in row-major order. */
void orc_elementwise(int op, int d, int is_f64, int rank, void* drn, const int32_t* drn_cfg, const void* a,
                     const int32_t* a_cfg, const void* b, const int32_t* b_cfg, int start, int end) {
    view_t v0 = view_of(drn_cfg, rank), v1 = view_of(a_cfg, rank), v2 = view_of(b_cfg, rank);
    int i0[ORC_MAX_RANK], i1[ORC_MAX_RANK], i2[ORC_MAX_RANK];
    indices_of_index(&v0, start, i0);
    indices_of_index(&v1, start, i1);
    indices_of_index(&v2, start, i2);
    for (int i = start; i < end; i++) {
        if (is_f64) ((double*)drn)[index_of_indices(&v0, i0)] =
            orc_bin_f64(0, op, d, ((const double*)a)[index_of_indices(&v1, i1)], ((const double*)b)[index_of_indices(&v2, i2)]);
        else ((float*)drn)[index_of_indices(&v0, i0)] =
            orc_bin_f32(0, op, d, ((const float*)a)[index_of_indices(&v1, i1)], ((const float*)b)[index_of_indices(&v2, i2)]);
        increment(i0, v0.shape, rank);
        increment(i1, v1.shape, rank);
        increment(i2, v2.shape, rank);
    }
}

/* CPUScalarBroadcast._workloadFor, J/backend/main/implementations/broadcast/CPUScalarBroadcast.java:28-75 */
void orc_scalarization(int op, int d, int is_f64, int rank, void* drn, const int32_t* drn_cfg, const void* src,
                       const int32_t* src_cfg, double value, int start, int end) {
    view_t v0 = view_of(drn_cfg, rank), v1 = view_of(src_cfg, rank);
    int i0[ORC_MAX_RANK], i1[ORC_MAX_RANK];
    indices_of_index(&v0, start, i0);
    indices_of_index(&v1, start, i1);
    for (int i = start; i < end; i++) {
        if (is_f64) ((double*)drn)[index_of_indices(&v0, i0)] = orc_bin_f64(1, op, d, ((const double*)src)[index_of_indices(&v1, i1)], value);
        else ((float*)drn)[index_of_indices(&v0, i0)] = orc_bin_f32(1, op, d, ((const float*)src)[index_of_indices(&v1, i1)], (float)value);
        increment(i0, v0.shape, rank);
        increment(i1, v1.shape, rank);
    }
}

/* ---- integer scalarization --------------------------------------------------------------------------------
 * java.lang.Math.round(double): "the closest long to the argument, with ties rounding to positive infinity";
 * NaN -> 0, at or beyond the ends of long -> Long.MIN_VALUE / Long.MAX_VALUE. */
static int64_t java_math_round(double a) {
    if (isnan(a)) return 0;
    if (a <= -9223372036854775808.0) return INT64_MIN;
    if (a >= 9223372036854775807.0) return INT64_MAX;
    double below = floor(a);
    if (a - below < 0.5) return (int64_t)below;       /* the difference is exact */
    return (int64_t)below + 1;
}
/* Java's narrowing primitive conversions (JLS 5.1.3) keep the low-order bits */
static int32_t to_int(int64_t v) { return (int32_t)(uint32_t)(uint64_t)v; }
static int16_t to_short(int64_t v) { return (int16_t)(uint16_t)(uint64_t)v; }
static int8_t to_byte(int64_t v) { return (int8_t)(uint8_t)(uint64_t)v; }
static int32_t int_neg(int32_t a) { return (int32_t)(0u - (uint32_t)a); }
static int64_t long_neg(int64_t a) { return (int64_t)(0ull - (uint64_t)a); }

/* the double overloads of the seven operator classes (family "scalar broadcast"): function, deriveAt0, deriveAt1.
 * CPUScalarBroadcastAddition.java, ...Subtraction, ...Multiplication, ...Division, ...Modulo, ...Identity,
 * CPUScalaBroadcastPower.java */
static double scalar_fun_f64(int op, int d, double a, double b) {
    switch (op) {
        case 0: return d < 0 ? a + b : 1;
        case 1: return d < 0 ? a - b : (d == 0 ? 1 : -1);
        case 2: return d < 0 ? a * b : (d == 0 ? b : a);
        case 3: return d < 0 ? a / b : (d == 0 ? 1 / b : -(a / orc_java_pow(b, 2)));
        case 4: return d < 0 ? fmod(a, b) : (d == 0 ? 1 / b : -(a / orc_java_pow(b, 2)));
        case 5: return d < 0 ? orc_java_pow(a, b) : (d == 0 ? b * orc_java_pow(a, b - 1) : orc_java_pow(a, b) * log(a));
        default: return b;
    }
}
/* invoke(int, int) of the same classes; returns 0 and sets *div_by_zero where Java throws ArithmeticException */
static int32_t scalar_fun_i32(int op, int d, int32_t a, int32_t b, int* div_by_zero) {
    switch (op) {
        case 0: return d < 0 ? (int32_t)((uint32_t)a + (uint32_t)b) : 1;
        case 1: return d < 0 ? (int32_t)((uint32_t)a - (uint32_t)b) : (d == 0 ? 1 : -1);
        case 2: return d < 0 ? (int32_t)((uint32_t)a * (uint32_t)b) : (d == 0 ? b : a);
        case 3: case 4:
            if (d < 0) {
                if (b == 0) { *div_by_zero = 1; return 0; }
                if (b == -1) return op == 3 ? int_neg(a) : 0;          /* JLS 15.17.2: MIN_VALUE / -1 overflows to MIN_VALUE */
                return op == 3 ? a / b : a % b;
            }
            if (d == 0) return to_int(java_math_round(1.0 / b));
            return to_int(java_math_round(int_neg(a) / orc_java_pow(b, 2)));
        case 5:
            if (d < 0) return to_int(java_math_round(orc_java_pow(a, b)));
            if (d == 0) return to_int(java_math_round(b * orc_java_pow(a, (int32_t)((uint32_t)b - 1u))));
            return to_int(java_math_round(orc_java_pow(a, b) * log(a)));
        default: return b;
    }
}
static int64_t scalar_fun_i64(int op, int d, int64_t a, int64_t b, int* div_by_zero) {
    switch (op) {
        case 0: return d < 0 ? (int64_t)((uint64_t)a + (uint64_t)b) : 1;
        case 1: return d < 0 ? (int64_t)((uint64_t)a - (uint64_t)b) : (d == 0 ? 1 : -1);
        case 2: return d < 0 ? (int64_t)((uint64_t)a * (uint64_t)b) : (d == 0 ? b : a);
        case 3: case 4:
            if (d < 0) {
                if (b == 0) { *div_by_zero = 1; return 0; }
                if (b == -1) return op == 3 ? long_neg(a) : 0;
                return op == 3 ? a / b : a % b;
            }
            if (d == 0) return java_math_round(1.0 / (double)b);
            return java_math_round((double)long_neg(a) / orc_java_pow((double)b, 2));
        case 5:
            if (d < 0) return java_math_round(orc_java_pow((double)a, (double)b));
            if (d == 0) return java_math_round((double)b * orc_java_pow((double)a, (double)(int64_t)((uint64_t)b - 1ull)));
            return java_math_round(orc_java_pow((double)a, (double)b) * log((double)a));
        default: return b;
    }
}

/* CPUScalarBroadcast._workloadFor for Integer / Long / Short / Byte (CPUScalarBroadcast.java:83-162).  Short has no
 * overload in any operator class and Byte only Identity's, so both run CPUBiFun's defaults (CPUBiFun.java:21-27):
 * (short) Math.round(invoke((double) a, (double) b)).  itype: 2 int, 3 long, 4 short, 5 byte.
 * Returns 1 where the CPU device throws ArithmeticException (nothing defined is written from there on). */
int orc_scalarization_int(int itype, int op, int d, int rank, void* drn, const int32_t* drn_cfg, const void* src,
                          const int32_t* src_cfg, int64_t number, int start, int end) {
    view_t v0 = view_of(drn_cfg, rank), v1 = view_of(src_cfg, rank);
    int i0[ORC_MAX_RANK], i1[ORC_MAX_RANK];
    int thrown = 0;
    indices_of_index(&v0, start, i0);
    indices_of_index(&v1, start, i1);
    for (int i = start; i < end && !thrown; i++) {
        int to = index_of_indices(&v0, i0), from = index_of_indices(&v1, i1);
        switch (itype) {
            case 2: ((int32_t*)drn)[to] = scalar_fun_i32(op, d, ((const int32_t*)src)[from], to_int(number), &thrown); break;
            case 3: ((int64_t*)drn)[to] = scalar_fun_i64(op, d, ((const int64_t*)src)[from], number, &thrown); break;
            case 4: ((int16_t*)drn)[to] = to_short(java_math_round(scalar_fun_f64(op, d, ((const int16_t*)src)[from], to_short(number)))); break;
            default: ((int8_t*)drn)[to] = op == 6 ? to_byte(number)
                                                  : to_byte(java_math_round(scalar_fun_f64(op, d, ((const int8_t*)src)[from], to_byte(number)))); break;
        }
        increment(i0, v0.shape, rank);
        increment(i1, v1.shape, rank);
    }
    return thrown;
}

/* CPUScalarBroadcastFunction (J/backend/main/implementations/scalar/CPUScalarBroadcastFunction.java:18-132):
 * drain[i] = value through the drain's view */
void orc_scalar_fill(int is_f64, int rank, void* drn, const int32_t* drn_cfg, double value, int start, int end) {
    view_t v0 = view_of(drn_cfg, rank);
    int i0[ORC_MAX_RANK];
    indices_of_index(&v0, start, i0);
    for (int i = start; i < end; i++) {
        if (is_f64) ((double*)drn)[index_of_indices(&v0, i0)] = value;
        else ((float*)drn)[index_of_indices(&v0, i0)] = (float)value;
        increment(i0, v0.shape, rank);
    }
}

/* CPUBroadcast._broadcastF32/_broadcastF64, J/backend/main/implementations/broadcast/CPUBroadcast.java:62-260,
 * loop for loop including the running/incrementing state machine of the reducing backward. */
#define BROADCAST_BODY(T, BIN)                                                                                   \
    view_t v0 = view_of(drn_cfg, rank), v1 = view_of(a_cfg, rank), v2 = view_of(b_cfg, rank);                    \
    const int32_t *t0Shp = v0.shape, *t1Shp = v1.shape, *t2Shp = v2.shape;                                       \
    int t0Idx[ORC_MAX_RANK], t1Idx[ORC_MAX_RANK], t2Idx[ORC_MAX_RANK];                                           \
    indices_of_index(&v0, i, t0Idx);                                                                             \
    indices_of_index(&v0, i, t1Idx);           /* t1Idx.set( t0_drn.indicesOfIndex( i ) ) */                     \
    for (int k = 0; k < rank; k++) t2Idx[k] = 0;                                                                 \
    T* t0_value = (T*)drn; const T* t1_value = (const T*)a; const T* t2_value = (const T*)b;                     \
    if (d < 0) {                                                                                                 \
        while (i < end) {                                                                                        \
            int ri = 0;                                                                                          \
            while (ri < rank) {                                                                                  \
                if (t1Shp[ri] == t2Shp[ri]) { t1Idx[ri] = t0Idx[ri]; t2Idx[ri] = t0Idx[ri]; }                    \
                else if (t1Shp[ri] > t2Shp[ri]) { t1Idx[ri] = t0Idx[ri]; t2Idx[ri] = 0; }                        \
                else if (t1Shp[ri] < t2Shp[ri]) { t1Idx[ri] = 0; t2Idx[ri] = t0Idx[ri]; }                        \
                ri++;                                                                                            \
            }                                                                                                    \
            t0_value[index_of_indices(&v0, t0Idx)] =                                                             \
                BIN(2, op, d, t1_value[index_of_indices(&v1, t1Idx)], t2_value[index_of_indices(&v2, t2Idx)]);   \
            increment(t0Idx, t0Shp, rank);                                                                       \
            i++;                                                                                                 \
        }                                                                                                        \
    } else {                                                                                                     \
        while (i < end) {                                                                                        \
            int ri = 0;                                                                                          \
            while (ri < rank) {                                                                                  \
                if (t0Shp[ri] == t1Shp[ri]) {                                                                    \
                    t1Idx[ri] = t0Idx[ri];                                                                       \
                    t2Idx[ri] = t0Idx[ri];                                                                       \
                    if (t2Shp[ri] == 1) t2Idx[ri] = 0; else t2Idx[ri] = t0Idx[ri];                               \
                } else if (t0Shp[ri] > t1Shp[ri]) { t1Idx[ri] = 0; t2Idx[ri] = t0Idx[ri]; }                      \
                ri++;                                                                                            \
            }                                                                                                    \
            T value = 0;                                                                                         \
            int running = 1, incrementing = 0;                                                                   \
            while (running) {                                                                                    \
                ri = (ri == rank ? 0 : ri);                                                                      \
                if (!incrementing) {                                                                             \
                    value += BIN(2, op, d, t1_value[index_of_indices(&v1, t1Idx)], t2_value[index_of_indices(&v2, t2Idx)]); \
                    incrementing = 1;                                                                            \
                    ri = 0;                                                                                      \
                } else {                                                                                         \
                    if (t0Shp[ri] < t1Shp[ri]) {                                                                 \
                        t1Idx[ri] = t1Idx[ri] + 1;                                                               \
                        t2Idx[ri] = t2Idx[ri] + 1;                                                               \
                        if (t1Idx[ri] == t1Shp[ri]) {                                                            \
                            t1Idx[ri] = 0; t2Idx[ri] = 0;                                                        \
                            running = (ri != rank - 1);                                                          \
                            ri++;                                                                                \
                        } else incrementing = 0;                                                                 \
                    } else { running = (ri != rank - 1); ri++; }                                                 \
                }                                                                                                \
            }                                                                                                    \
            t0_value[index_of_indices(&v0, t0Idx)] = value;                                                      \
            increment(t0Idx, t0Shp, rank);                                                                       \
            i++;                                                                                                 \
        }                                                                                                        \
    }

void orc_broadcast(int op, int d, int is_f64, int rank, void* drn, const int32_t* drn_cfg, const void* a,
                   const int32_t* a_cfg, const void* b, const int32_t* b_cfg, int i, int end) {
    if (is_f64) { BROADCAST_BODY(double, orc_bin_f64) }
    else { BROADCAST_BODY(float, orc_bin_f32) }
}

/* AbstractCPUConvolution._convolve32/_convolve64, J/backend/main/implementations/convolution/AbstractCPUConvolution.java:70-143,245-316 */
#define CONVOLVE_BODY(T)                                                                                         \
    view_t v0 = view_of(drn_cfg, rank), v1 = view_of(a_cfg, rank), v2 = view_of(b_cfg, rank);                    \
    int t0Idx[ORC_MAX_RANK], t1Idx[ORC_MAX_RANK] = {0}, t2Idx[ORC_MAX_RANK] = {0};                               \
    indices_of_index(&v0, start, t0Idx);                                                                         \
    T* t0_value = (T*)drn; const T* t1_value = (const T*)a; const T* t2_value = (const T*)b;                     \
    int i = start;                                                                                               \
    while (i < end) {                                                                                            \
        int ri = 0;                                                                                              \
        while (ri < rank) {                                                                                      \
            if (v1.shape[ri] == v2.shape[ri]) { t1Idx[ri] = t0Idx[ri]; t2Idx[ri] = t0Idx[ri]; }                  \
            else if (v1.shape[ri] > v2.shape[ri]) { t1Idx[ri] = t0Idx[ri]; t2Idx[ri] = 0; }                      \
            else if (v1.shape[ri] < v2.shape[ri]) { t1Idx[ri] = 0; t2Idx[ri] = t0Idx[ri]; }                      \
            ri++;                                                                                                \
        }                                                                                                        \
        T value = 0;                                                                                             \
        int running = 1, incrementing = 0;                                                                       \
        while (running) {                                                                                        \
            ri = (ri == rank ? 0 : ri);                                                                          \
            if (!incrementing) {                                                                                 \
                value += t1_value[index_of_indices(&v1, t1Idx)] * t2_value[index_of_indices(&v2, t2Idx)];        \
                incrementing = 1;                                                                                \
                ri = 0;                                                                                          \
            } else {                                                                                             \
                if (t1Idx[ri] < v1.shape[ri] && t2Idx[ri] < v2.shape[ri]) {                                      \
                    t1Idx[ri] = t1Idx[ri] + 1;                                                                   \
                    t2Idx[ri] = t2Idx[ri] + 1;                                                                   \
                    if (t1Idx[ri] == v1.shape[ri] || t2Idx[ri] == v2.shape[ri]) {                                \
                        running = (ri != rank - 1);                                                              \
                        if (v1.shape[ri] == v2.shape[ri]) { t1Idx[ri] = t0Idx[ri]; t2Idx[ri] = t0Idx[ri]; }      \
                        else if (v1.shape[ri] > v2.shape[ri]) { t1Idx[ri] = t0Idx[ri]; t2Idx[ri] = 0; }          \
                        else if (v1.shape[ri] < v2.shape[ri]) { t1Idx[ri] = 0; t2Idx[ri] = t0Idx[ri]; }          \
                        ri++;                                                                                    \
                    } else incrementing = 0;                                                                     \
                } else ri++;                                                                                     \
            }                                                                                                    \
        }                                                                                                        \
        t0_value[index_of_indices(&v0, t0Idx)] = value;                                                          \
        increment(t0Idx, v0.shape, rank);                                                                        \
        i++;                                                                                                     \
    }

void orc_convolve(int is_f64, int rank, void* drn, const int32_t* drn_cfg, const void* a, const int32_t* a_cfg,
                  const void* b, const int32_t* b_cfg, int start, int end) {
    if (is_f64) { CONVOLVE_BODY(double) }
    else { CONVOLVE_BODY(float) }
}

/* AbstractCPUConvolution._deConvolve32/_deConvolve64, AbstractCPUConvolution.java:146-240,319-408.
 * (The "incrementing if i>0" prologue of the reference only re-derives t1Idx from t0Idx/t2Idx, which
 * the main loop does again for every element; it has no effect on results and is restated as is.) */
#define DECONVOLVE_BODY(T)                                                                                       \
    view_t v0 = view_of(drn_cfg, rank), v1 = view_of(a_cfg, rank), v2 = view_of(b_cfg, rank);                    \
    int t0Idx[ORC_MAX_RANK], t1Idx[ORC_MAX_RANK] = {0}, t2Idx[ORC_MAX_RANK] = {0};                               \
    indices_of_index(&v0, start, t0Idx);                                                                         \
    T* t0_value = (T*)drn; const T* t1_value = (const T*)a; const T* t2_value = (const T*)b;                     \
    for (int ii = 0; ii < start; ii++) {                                                                         \
        int ri = 0;                                                                                              \
        while (ri < rank) {                                                                                      \
            if (t2Idx[ri] == v2.shape[ri]) { t1Idx[ri] = t0Idx[ri]; t2Idx[ri] = 0; }                             \
            else t1Idx[ri] = v0.shape[ri] > v1.shape[ri] ? (t0Idx[ri] - t2Idx[ri]) : (t0Idx[ri] + t2Idx[ri]);    \
            ri++;                                                                                                \
        }                                                                                                        \
    }                                                                                                            \
    int i = start;                                                                                               \
    while (i < end) {                                                                                            \
        int ri = 0;                                                                                              \
        while (ri < rank) {                                                                                      \
            if (t2Idx[ri] == v2.shape[ri]) { t1Idx[ri] = t0Idx[ri]; t2Idx[ri] = 0; }                             \
            else t1Idx[ri] = (v0.shape[ri] > v1.shape[ri]) ? (t0Idx[ri] - t2Idx[ri]) : (t0Idx[ri] + t2Idx[ri]);  \
            ri++;                                                                                                \
        }                                                                                                        \
        T value = 0;                                                                                             \
        int running = 1, incrementing = 0;                                                                       \
        while (running) {                                                                                        \
            ri = (ri == rank ? 0 : ri);                                                                          \
            if (!incrementing) {                                                                                 \
                int isMatch = 1;                                                                                 \
                for (int rii = 0; rii < rank; rii++)                                                             \
                    isMatch = (t1Idx[rii] < v1.shape[rii] && t1Idx[rii] >= 0) && isMatch;                        \
                value += (isMatch ? t1_value[index_of_indices(&v1, t1Idx)] * t2_value[index_of_indices(&v2, t2Idx)] : 0); \
                incrementing = 1;                                                                                \
                ri = 0;                                                                                          \
            } else {                                                                                             \
                if (t2Idx[ri] < v2.shape[ri]) {                                                                  \
                    t2Idx[ri] = t2Idx[ri] + 1;                                                                   \
                    if (t2Idx[ri] == v2.shape[ri]) {                                                             \
                        running = (ri != rank - 1);                                                              \
                        t1Idx[ri] = t0Idx[ri];                                                                   \
                        t2Idx[ri] = 0;                                                                           \
                        ri++;                                                                                    \
                    } else {                                                                                     \
                        t1Idx[ri] = v0.shape[ri] > v1.shape[ri] ? (t0Idx[ri] - t2Idx[ri]) : (t0Idx[ri] + t2Idx[ri]); \
                        incrementing = 0;                                                                        \
                    }                                                                                            \
                } else ri++;                                                                                     \
            }                                                                                                    \
        }                                                                                                        \
        t0_value[index_of_indices(&v0, t0Idx)] = value;                                                          \
        increment(t0Idx, v0.shape, rank);                                                                        \
        i++;                                                                                                     \
    }

void orc_deconvolve(int is_f64, int rank, void* drn, const int32_t* drn_cfg, const void* a, const int32_t* a_cfg,
                    const void* b, const int32_t* b_cfg, int start, int end) {
    if (is_f64) { DECONVOLVE_BODY(double) }
    else { DECONVOLVE_BODY(float) }
}

/* The same gradient with the loop restricted to the error entries that can pass the bounds test.
 * Skipped iterations add +0 to a sum that is never -0, so the result is bit-identical to
 * orc_deconvolve (tests check that on small shapes); this is what makes the full-size gradient of
 * [64,256,256] checkable in seconds instead of the 2.7e11 iterations of the literal loop. */
#define DECONVOLVE_FAST_BODY(T)                                                                                  \
    view_t v0 = view_of(drn_cfg, rank), v1 = view_of(a_cfg, rank), v2 = view_of(b_cfg, rank);                    \
    int o[ORC_MAX_RANK];                                                                                         \
    indices_of_index(&v0, start, o);                                                                             \
    for (int i = start; i < end; i++) {                                                                          \
        int lo[ORC_MAX_RANK], hi[ORC_MAX_RANK], e[ORC_MAX_RANK], i1[ORC_MAX_RANK], empty = 0;                    \
        for (int k = 0; k < rank; k++) {                                                                         \
            if (v0.shape[k] > v1.shape[k]) {                                                                     \
                lo[k] = o[k] - v1.shape[k] + 1; if (lo[k] < 0) lo[k] = 0;                                        \
                hi[k] = o[k] + 1; if (hi[k] > v2.shape[k]) hi[k] = v2.shape[k];                                  \
            } else {                                                                                             \
                lo[k] = 0;                                                                                       \
                hi[k] = v1.shape[k] - o[k]; if (hi[k] > v2.shape[k]) hi[k] = v2.shape[k];                        \
            }                                                                                                    \
            if (hi[k] <= lo[k]) empty = 1;                                                                       \
            e[k] = lo[k];                                                                                        \
        }                                                                                                        \
        T value = 0;                                                                                             \
        int running = !empty;                                                                                    \
        while (running) {                                                                                        \
            for (int k = 0; k < rank; k++) i1[k] = v0.shape[k] > v1.shape[k] ? o[k] - e[k] : o[k] + e[k];        \
            value += ((const T*)a)[index_of_indices(&v1, i1)] * ((const T*)b)[index_of_indices(&v2, e)];         \
            int k = 0;                                                                                           \
            for (; k < rank; k++) { if (++e[k] < hi[k]) break; e[k] = lo[k]; }                                   \
            running = k < rank;                                                                                  \
        }                                                                                                        \
        ((T*)drn)[index_of_indices(&v0, o)] = value;                                                             \
        increment(o, v0.shape, rank);                                                                            \
    }

void orc_deconvolve_fast(int is_f64, int rank, void* drn, const int32_t* drn_cfg, const void* a, const int32_t* a_cfg,
                         const void* b, const int32_t* b_cfg, int start, int end) {
    if (is_f64) { DECONVOLVE_FAST_BODY(double) }
    else { DECONVOLVE_FAST_BODY(float) }
}

/* SimpleCPUConvolution.ImplF32/ImplF64.run(batchIndex), J/backend/main/implementations/convolution/SimpleCPUConvolution.java:143-159,217-233 */
void orc_simple_conv2d(int is_f64, const void* image, const void* kernel, void* result, int width, int height,
                       int kernelWidth, int kernelHeight, int batchIndex) {
    int resultWidth = width - kernelWidth + 1, resultHeight = height - kernelHeight + 1;
    int imageOffset = batchIndex * width * height;
    int resultOffset = batchIndex * resultWidth * resultHeight;
    for (int y = 0; y < resultHeight; y++)
        for (int x = 0; x < resultWidth; x++) {
            if (is_f64) {
                double sum = 0;
                for (int ky = 0; ky < kernelHeight; ky++)
                    for (int kx = 0; kx < kernelWidth; kx++)
                        sum += ((const double*)image)[imageOffset + (y + ky) * width + (x + kx)] * ((const double*)kernel)[ky * kernelWidth + kx];
                ((double*)result)[resultOffset + y * resultWidth + x] = sum;
            } else {
                float sum = 0;
                for (int ky = 0; ky < kernelHeight; ky++)
                    for (int kx = 0; kx < kernelWidth; kx++)
                        sum += ((const float*)image)[imageOffset + (y + ky) * width + (x + kx)] * ((const float*)kernel)[ky * kernelWidth + kx];
                ((float*)result)[resultOffset + y * resultWidth + x] = sum;
            }
        }
}

/* CPUSum._runRecursively, J/backend/main/operations/other/internal/CPUSum.java:26-74: tiles of RTS = 128 elements are
 * summed front to back into a value that starts at 0; the partial sums are reduced the same way until one is left. */
double orc_sum_tree(int is_f64, const void* data, int size) {
    const int RTS = 128;
    if (size == 1) return is_f64 ? ((const double*)data)[0] : (double)((const float*)data)[0];
    int N = (size + RTS - 1) / RTS;
    double result;
    if (is_f64) {
        double* out = (double*)malloc(sizeof(double) * (size_t)N);
        for (int ni = 0; ni < N; ni++) {
            int offset = ni * RTS, limit = offset + RTS < size ? offset + RTS : size;
            double value = 0;
            for (int i = offset; i < limit; ++i) value += ((const double*)data)[i];
            out[ni] = value;
        }
        result = N > 1 ? orc_sum_tree(1, out, N) : out[0];
        free(out);
    } else {
        float* out = (float*)malloc(sizeof(float) * (size_t)N);
        for (int ni = 0; ni < N; ni++) {
            int offset = ni * RTS, limit = offset + RTS < size ? offset + RTS : size;
            float value = 0;
            for (int i = offset; i < limit; ++i) value += ((const float*)data)[i];
            out[ni] = value;
        }
        result = N > 1 ? orc_sum_tree(0, out, N) : (double)out[0];
        free(out);
    }
    return result;
}

/* CPUReduce._runRecursively, J/backend/main/operations/other/internal/CPUReduce.java:90-157: per tile of RTS = 64
 * the index of the first element that beats (strictly) everything before it; the winners are gathered and reduced
 * the same way; the result is an index into the original data.  type 0 = MIN, 1 = MAX. */
int orc_reduce_index(int type, int is_f64, const void* data, int size) {
    const int RTS = 64;
    int N = (size + RTS - 1) / RTS;
    if (size == 1) return 0;
    int* out = (int*)malloc(sizeof(int) * (size_t)N);
    for (int ni = 0; ni < N; ni++) {
        int offset = ni * RTS, limit = offset + RTS < size ? offset + RTS : size;
        int found_index = offset;
        if (is_f64) {
            double value = ((const double*)data)[offset];
            for (int i = offset + 1; i < limit; ++i) {
                double current = ((const double*)data)[i];
                if (type == 0 ? current < value : current > value) { value = current; found_index = i; }
            }
        } else {
            float value = ((const float*)data)[offset];
            for (int i = offset + 1; i < limit; ++i) {
                float current = ((const float*)data)[i];
                if (type == 0 ? current < value : current > value) { value = current; found_index = i; }
            }
        }
        out[ni] = found_index;
    }
    int result = out[0];
    if (N > 1) {
        size_t es = is_f64 ? sizeof(double) : sizeof(float);
        char* reduced = (char*)malloc(es * (size_t)N);
        for (int i = 0; i < N; i++) memcpy(reduced + es * (size_t)i, (const char*)data + es * (size_t)out[i], es);
        result = out[orc_reduce_index(type, is_f64, reduced, N)];
        free(reduced);
    }
    free(out);
    return result;
}

/* DOT.unrolled04, J/backend/main/operations/linear/internal/blas/DOT.java (float and double overloads): four running
 * sums over every fourth element, the remainder into the first, added left to right; products are rounded. */
double orc_dot(int is_f64, const void* a, const void* b, int size) {
    int remainder = size % 4, i = 0;
    if (is_f64) {
        const double *x = (const double*)a, *y = (const double*)b;
        double sum0 = 0, sum1 = 0, sum2 = 0, sum3 = 0;
        for (int lim = size - remainder; i < lim; i += 4) {
            sum0 += x[i] * y[i]; sum1 += x[i + 1] * y[i + 1]; sum2 += x[i + 2] * y[i + 2]; sum3 += x[i + 3] * y[i + 3];
        }
        for (; i < size; i++) sum0 += x[i] * y[i];
        return sum0 + sum1 + sum2 + sum3;
    } else {
        const float *x = (const float*)a, *y = (const float*)b;
        float sum0 = 0, sum1 = 0, sum2 = 0, sum3 = 0;
        for (int lim = size - remainder; i < lim; i += 4) {
            sum0 += x[i] * y[i]; sum1 += x[i + 1] * y[i + 1]; sum2 += x[i + 2] * y[i + 2]; sum3 += x[i + 3] * y[i + 3];
        }
        for (; i < size; i++) sum0 += x[i] * y[i];
        return (double)(sum0 + sum1 + sum2 + sum3);
    }
}

/* GEMM.partial_F32_MxN_RM / partial_F64_MxN_RM and the CM twins with AXPY inlined:
 * J/backend/main/operations/linear/internal/blas/GEMM.java:258-304, AXPY.java:32-59.
 * [first, limit) is a range of rows of A (row major) or of columns of B (column major). */
void orc_gemm_partial(int is_f64, int row_major, void* product, int first, int limit, const void* left, int left_len,
                      int complexity, const void* right, int right_len) {
    if (row_major) {
        int rightCols = right_len / complexity;
        for (int c = 0; c < complexity; c++)
            for (int j = first; j < limit; j++) {
                if (is_f64) {
                    double* y = (double*)product + j * rightCols; const double* x = (const double*)right + c * rightCols;
                    double a = ((const double*)left)[c + j * complexity];
                    for (int i = 0; i < rightCols; i++) y[i] += a * x[i];
                } else {
                    float* y = (float*)product + j * rightCols; const float* x = (const float*)right + c * rightCols;
                    float a = ((const float*)left)[c + j * complexity];
                    for (int i = 0; i < rightCols; i++) y[i] += a * x[i];
                }
            }
    } else {
        int nbRows = left_len / complexity;
        for (int c = 0; c < complexity; c++)
            for (int j = first; j < limit; j++) {
                if (is_f64) {
                    double* y = (double*)product + j * nbRows; const double* x = (const double*)left + c * nbRows;
                    double a = ((const double*)right)[c + j * complexity];
                    for (int i = 0; i < nbRows; i++) y[i] += a * x[i];
                } else {
                    float* y = (float*)product + j * nbRows; const float* x = (const float*)left + c * nbRows;
                    float a = ((const float*)right)[c + j * complexity];
                    for (int i = 0; i < nbRows; i++) y[i] += a * x[i];
                }
            }
    }
}

/* ------------------------------------------------------------------------------------------------
 * Seeded generator: CPURandomization.gaussianFrom/_nextSeed/_nextDouble
 * (J/backend/main/implementations/elementwise/CPURandomization.java:139-153,263-323) and
 * Arg.Seed._longStringHash (J/math/args/Arg.java:96-102).
 */
static const int64_t RNG_MULTIPLIER = 0x5DEECE66DLL, RNG_ADDEND = 0xBLL, RNG_MASK = (1LL << 48) - 1;

int64_t orc_long_string_hash(const char* s) {
    uint64_t h = 1125899906842597ULL;
    for (; *s; s++) h = 31 * h + (unsigned char)*s;
    return (int64_t)h;
}

int64_t orc_initial_scramble(int64_t seed) { return (seed ^ RNG_MULTIPLIER) & RNG_MASK; }

static int64_t next_seed(int64_t currentSeed) {
    int64_t oldseed, nextseed;
    do {
        oldseed = currentSeed;
        nextseed = (int64_t)(((uint64_t)oldseed * (uint64_t)RNG_MULTIPLIER + (uint64_t)RNG_ADDEND) & (uint64_t)RNG_MASK);
    } while (oldseed == (currentSeed = nextseed));
    return nextseed;
}
static int32_t next_bits(int bits, int64_t seed) { return (int32_t)((uint64_t)seed >> (48 - bits)); }
static double next_double(int64_t seed1, int64_t seed2) {
    return (double)(((int64_t)next_bits(26, seed1) << 27) + next_bits(27, seed2)) * 0x1.0p-53;
}

void orc_gaussian_from(int64_t seed, double* out) {
    double v1, v2, s;
    do {
        int64_t seed1 = next_seed(seed), seed2 = next_seed(seed1), seed3 = next_seed(seed2), seed4 = next_seed(seed3);
        v1 = 2 * next_double(seed1, seed2) - 1;
        v2 = 2 * next_double(seed3, seed4) - 1;
        s = v1 * v1 + v2 * v2;
        seed = seed4;
    } while (s >= 1 || s == 0);
    double multiplier = sqrt(-2 * log(s) / s);     /* StrictMath in the reference */
    out[0] = v1 * multiplier;
    out[1] = v2 * multiplier;
}

/* the simple (contiguous) f32/f64 workloads of CPURandomization.java:108-153 */
void orc_fill_gaussian(int is_f64, void* data, int64_t seed, int i, int end) {
    double g[2] = {0, 0};
    if (i % 2 == 1) {
        orc_gaussian_from(seed + i - 1, g);
        if (is_f64) ((double*)data)[i] = g[1]; else ((float*)data)[i] = (float)g[1];
        i++;
    }
    for (; i < end; i += 2) {
        orc_gaussian_from(seed + i, g);
        if (is_f64) { ((double*)data)[i] = g[0]; if (i + 1 < end) ((double*)data)[i + 1] = g[1]; }
        else { ((float*)data)[i] = (float)g[0]; if (i + 1 < end) ((float*)data)[i + 1] = (float)g[1]; }
    }
}

/* ------------------------------------------------------------------------------------------------
 * CPU.JVMExecutor.threaded + WorkScheduler.Divider: split [first, limit) in halves while more than one
 * worker is left and the range is above the threshold, run the leaves concurrently
 * (J/devices/host/CPU.java:743-797; J/devices/host/concurrent/WorkScheduler.java:132-159).
 */
typedef void (*orc_range_fn)(void* ctx, int start, int end);
typedef struct { orc_range_fn fn; void* ctx; int first, limit, workers, threshold; } split_t;

static void* split_run(void* p) {
    split_t* s = (split_t*)p;
    int count = s->limit - s->first;
    if (count > s->threshold && s->workers > 1) {
        int split = s->first + count / 2;
        int nextWorkers = s->workers / 2;
        split_t lo = {s->fn, s->ctx, s->first, split, nextWorkers, s->threshold};
        split_t hi = {s->fn, s->ctx, split, s->limit, nextWorkers, s->threshold};
        pthread_t th;
        int spawned = pthread_create(&th, NULL, split_run, &lo) == 0;
        if (!spawned) split_run(&lo);
        split_run(&hi);
        if (spawned) pthread_join(th, NULL);
    } else s->fn(s->ctx, s->first, s->limit);
    return NULL;
}

void orc_threaded(orc_range_fn fn, void* ctx, int first, int limit, int workers, int threshold) {
    split_t s = {fn, ctx, first, limit, workers, threshold};
    split_run(&s);
}

/* leaf ranges the splitter produces, for tests: writes up to cap (start, end) pairs, returns the count */
typedef struct { int* out; int cap; int n; pthread_mutex_t mu; } leaves_t;
static void record_leaf(void* ctx, int start, int end) {
    leaves_t* l = (leaves_t*)ctx;
    pthread_mutex_lock(&l->mu);
    if (l->n < l->cap) { l->out[2 * l->n] = start; l->out[2 * l->n + 1] = end; }
    l->n++;
    pthread_mutex_unlock(&l->mu);
}
int orc_split_leaves(int first, int limit, int workers, int threshold, int* out, int cap) {
    leaves_t l = {out, cap, 0, PTHREAD_MUTEX_INITIALIZER};
    orc_threaded(record_leaf, &l, first, limit, workers, threshold);
    return l.n;
}

/* threaded wrappers used by the CPU-baseline timing (same kernels, scheduled like the reference) */
typedef struct {
    int kind, op, d, is_f64, rank;
    void* drn; const int32_t* drn_cfg; const void* a; const int32_t* a_cfg; const void* b; const int32_t* b_cfg;
    double value;
    int left_len, complexity, right_len, row_major;
} job_t;

static void job_run(void* ctx, int start, int end) {
    job_t* j = (job_t*)ctx;
    switch (j->kind) {
        case 0: orc_activation(j->op, j->d, j->is_f64, j->rank, j->drn, j->drn_cfg, j->a, j->a_cfg, start, end); break;
        case 1: orc_elementwise(j->op, j->d, j->is_f64, j->rank, j->drn, j->drn_cfg, j->a, j->a_cfg, j->b, j->b_cfg, start, end); break;
        case 2: orc_scalarization(j->op, j->d, j->is_f64, j->rank, j->drn, j->drn_cfg, j->a, j->a_cfg, j->value, start, end); break;
        case 3: orc_broadcast(j->op, j->d, j->is_f64, j->rank, j->drn, j->drn_cfg, j->a, j->a_cfg, j->b, j->b_cfg, start, end); break;
        case 4: orc_convolve(j->is_f64, j->rank, j->drn, j->drn_cfg, j->a, j->a_cfg, j->b, j->b_cfg, start, end); break;
        case 5: orc_deconvolve(j->is_f64, j->rank, j->drn, j->drn_cfg, j->a, j->a_cfg, j->b, j->b_cfg, start, end); break;
        case 6: orc_deconvolve_fast(j->is_f64, j->rank, j->drn, j->drn_cfg, j->a, j->a_cfg, j->b, j->b_cfg, start, end); break;
        case 7: orc_gemm_partial(j->is_f64, j->row_major, j->drn, start, end, j->a, j->left_len, j->complexity, j->b, j->right_len); break;
    }
}

/* kind: 0 activation, 1 elementwise, 2 scalarization, 3 broadcast, 4 convolve, 5 deconvolve, 6 deconvolve_fast.
 * Runs over [first, limit) of the drain's flat index with the reference's splitter (threshold 32, CPU.java:748). */
void orc_run_threaded(int kind, int op, int d, int is_f64, int rank, void* drn, const int32_t* drn_cfg, const void* a,
                      const int32_t* a_cfg, const void* b, const int32_t* b_cfg, double value, int first, int limit, int workers) {
    job_t j = {kind, op, d, is_f64, rank, drn, drn_cfg, a, a_cfg, b, b_cfg, value, 0, 0, 0, 0};
    orc_threaded(job_run, &j, first, limit, workers, 32);
}

/* GEMM.threaded_F32_MxN_RM / _CM (GEMM.java:306-335): rows of A (RM) or columns of B (CM) split like any workload */
void orc_gemm_threaded(int is_f64, int row_major, void* product, const void* left, int left_len, int complexity,
                       const void* right, int right_len, int workers) {
    job_t j = {7, 0, 0, is_f64, 0, product, NULL, left, NULL, right, NULL, 0.0, left_len, complexity, right_len, row_major};
    int count = row_major ? left_len / complexity : right_len / complexity;
    orc_threaded(job_run, &j, 0, count, workers, 32);
}
