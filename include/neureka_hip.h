/*
 * neureka_hip.h — C ABI of libneureka_hip.so, the native half of a `HipDevice` for Neureka.
 *
 * Every entry point replaces one JOCL/OpenCL call site (or one family of kernel launches) of the
 * reference's OpenCLDevice.  Citations are relative to the reference tree:
 *   J/ = src/main/java/neureka/      K/ = src/main/resources/kernels/
 *
 * Conventions
 *   - Every function returns 0 on success and a non-zero status otherwise (HIP error code, or one of
 *     the NK_ERR_* values); nk_last_error() gives the message of the last failure on this thread.
 *   - nk_dev is an opaque device handle; nk_buf is a device address (a Java `long`), valid until
 *     nk_free.  Host memory is never owned by the library.
 *   - One in-order HIP stream per device.  nk_h2d / nk_d2h / nk_device_sync return after the work
 *     is complete (the reference uses blocking CL_TRUE transfers: J/devices/opencl/OpenCLDevice.java:446,488,626,678);
 *     kernel launches are asynchronous and ordered on that stream.
 *   - A view descriptor ("cfg") is NDConfiguration.asInlineArray(): int32[5*rank] laid out as
 *     shape | strides | indicesMap | offset | spread   (J/ndim/config/NDConfiguration.java:335-345).
 *     Descriptors are passed by value with each launch (kernel arguments), there is no device-side
 *     descriptor cache like OpenCLDevice.clConfigOf (J/devices/opencl/OpenCLDevice.java:418-456).
 *     rank <= NK_MAX_RANK.
 *   - `d` is the derivative index of the ExecutionCall (Arg.DerivIdx), -1 = forward.
 *   - `n` is the drain's element count (the OpenCL global work size), < 2^31 like a Java int.
 *   - dtype: NK_F32 or NK_F64.  Slot order follows the reference: drain first, then sources.
 *   - Calls on one device handle from several host threads are serialised inside the library (a lock per device
 *     held for the length of a call), so they are safe but do not overlap; nk_last_error / nk_last_path are per thread.
 *     A handle closed while another thread waits for it makes that call fail with NK_ERR_HANDLE.
 */
#ifndef NEUREKA_HIP_H
#define NEUREKA_HIP_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint64_t nk_dev;
typedef uint64_t nk_buf;

#define NK_MAX_RANK 8

enum { NK_F32 = 0, NK_F64 = 1,
       NK_I32 = 2, NK_I64 = 3, NK_I16 = 4, NK_I8 = 5 };   /* integer types: nk_scalarization_int only */

/* status codes besides hipError_t values */
enum {
    NK_OK = 0,
    NK_ERR_ARG = 10001,         /* malformed argument (null pointer, bad rank/dtype/id, size mismatch) */
    NK_ERR_UNSUPPORTED = 10002, /* well-formed but not implemented on this device */
    NK_ERR_HANDLE = 10003       /* unknown device or buffer handle */
};

/* binary operator ids: the operation identifiers the reference splices into its kernel names
 * (J/backend/main/implementations/ParsedCLImplementation.java:17-37; J/backend/ocl/CLBackend.java:200-260) */
enum {
    NK_OP_ADD = 0, NK_OP_SUB = 1, NK_OP_MUL = 2, NK_OP_DIV = 3, NK_OP_MOD = 4, NK_OP_POW = 5,
    NK_OP_IDY = 6  /* scalarization only: drain = value (CLScalarBroadcastIdentity) */
};

/* unary function ids: ScalarFun.id() of J/backend/main/implementations/fun/api/ScalarFun.java:7-31 */
enum {
    NK_FUN_ABS = 0, NK_FUN_COS, NK_FUN_GASU, NK_FUN_GATU, NK_FUN_GAUS, NK_FUN_FAST_GAUS, NK_FUN_GELU,
    NK_FUN_IDY, NK_FUN_LN, NK_FUN_QUAD, NK_FUN_RELU, NK_FUN_SELU, NK_FUN_SIG, NK_FUN_SILU, NK_FUN_SIN,
    NK_FUN_SOFTPLUS, NK_FUN_SOFTSIGN, NK_FUN_TANH, NK_FUN_FAST_TANH, NK_FUN_EXP, NK_FUN_LOG10,
    NK_FUN_SQRT, NK_FUN_CBRT, NK_FUN_COUNT
};

enum { NK_LAYOUT_ROW_MAJOR = 0, NK_LAYOUT_COLUMN_MAJOR = 1 };

const char* nk_last_error(void);
/* Names one of the kernel paths chosen by the last launch on this thread ("contiguous", "rows", "tile_transpose",
 * "generic", "mfma", ...).  Diagnostic only; lets tests assert that a fast path was really taken. */
const char* nk_last_path(void);

/* ---- lifecycle: replaces clGetPlatformIDs/clGetDeviceIDs/clCreateContext/clCreateCommandQueue
 *      (J/backend/ocl/CLBackend.java:96-152, J/devices/opencl/OpenCLPlatform.java:60-101) and
 *      clFinish + clReleaseCommandQueue on dispose (J/devices/opencl/OpenCLDevice.java:299-304). */
int nk_device_count(int* count);
int nk_device_open(int index, nk_dev* dev);
int nk_device_close(nk_dev dev);           /* frees every buffer still alive on the device */
int nk_device_sync(nk_dev dev);
/* device properties: J/devices/opencl/OpenCLDevice.java:738-809 (name, globalMemSize, maxComputeUnits, ...) */
int nk_device_props(nk_dev dev, char* name, size_t name_cap, int* compute_units, int* clock_mhz,
                    uint64_t* global_mem_bytes, int* lds_bytes_per_block, int* wavefront_size);
/* memory of the device that is free right now, and all of it (the latter is CL_DEVICE_GLOBAL_MEM_SIZE,
 * J/devices/opencl/OpenCLDevice.java:770-774; the former has no counterpart in the reference).  Blocks at rest in
 * the pool count as used: the driver does not know they are free. */
int nk_device_memory(nk_dev dev, uint64_t* free_bytes, uint64_t* total_bytes);
/* live-allocation accounting, what numberOfDataObjects()-style leak tests observe
 * (J/devices/AbstractDeviceData.java:24-56) */
int nk_device_stats(nk_dev dev, uint64_t* live_buffers, uint64_t* live_bytes);

/* ---- memory: clCreateBuffer (OpenCLDevice.java:439,465), clReleaseMemObject (:454,957-962),
 *      clEnqueueWriteBuffer (:446,488,626), clEnqueueReadBuffer (:678), clEnqueueFillBuffer (:481). */
int nk_alloc(nk_dev dev, uint64_t bytes, nk_buf* buf);
int nk_free(nk_dev dev, nk_buf buf);
int nk_h2d(nk_dev dev, nk_buf dst, uint64_t dst_byte_off, const void* host, uint64_t bytes);
int nk_d2h(nk_dev dev, void* host, nk_buf src, uint64_t src_byte_off, uint64_t bytes);
int nk_d2d(nk_dev dev, nk_buf dst, uint64_t dst_byte_off, nk_buf src, uint64_t src_byte_off, uint64_t bytes);
/* writes `count` copies of a 1/2/4/8-byte pattern starting at dst + dst_byte_off */
int nk_fill(nk_dev dev, nk_buf dst, uint64_t dst_byte_off, const void* pattern, int pattern_bytes, uint64_t count);

/* ---- the buffer pool behind nk_alloc / nk_free.  No counterpart in the reference, whose clCreateBuffer and
 *      clReleaseMemObject go to the driver for every tensor (OpenCLDevice.java:465,957-962).  nk_free keeps the block, by
 *      size class, for the next nk_alloc and neither call waits for the device: the one in-order stream orders the work of
 *      a block's successive owners.  nk_alloc returns memory with arbitrary contents, like clCreateBuffer.  Blocks at rest
 *      go back to the driver when they would exceed the limit (default: half of the device's memory), when the driver
 *      runs out of memory, on nk_pool_trim and on nk_device_close. */
int nk_pool_trim(nk_dev dev);
int nk_pool_stats(nk_dev dev, uint64_t* resting_blocks, uint64_t* resting_bytes, uint64_t* driver_allocations, uint64_t* reuses);
/* max_resting_bytes: the limit above.  poison != 0: every block is handed out filled with 0xFF bytes (NaN as float or
 * double), for tests that prove that no operation relies on the contents of a fresh buffer. */
int nk_pool_config(nk_dev dev, uint64_t max_resting_bytes, int poison);

/* ---- timing on the device stream (no counterpart in the reference, which only measures wall clock
 *      around closures: src/test/java/testutility/Measure.java).  Events are recorded on the device's
 *      own stream so that they bracket exactly the launches made through this library. */
int nk_event_create(nk_dev dev, uint64_t* event);
int nk_event_record(nk_dev dev, uint64_t event);
int nk_event_elapsed_ms(nk_dev dev, uint64_t start, uint64_t stop, float* ms); /* synchronises on `stop` */
int nk_event_destroy(nk_dev dev, uint64_t event);

/* ---- kernels -------------------------------------------------------------------------------- */

/* activation_<fun>: K/activation_template.cl:23-45, launched by
 * J/backend/main/implementations/elementwise/CLElementwiseFunction.java:27-41.
 * drain[i] = f(src[i]) for d < 0, f'(src[i]) for d >= 0.  CPU semantics:
 * J/backend/main/implementations/elementwise/CPUElementwiseFunction.java:18-117. */
int nk_activation(nk_dev dev, int fun_id, int d, int dtype, int rank,
                  nk_buf drn, const int32_t* drn_cfg, nk_buf src, const int32_t* src_cfg, int64_t n);

/* elementwise_<op>: K/elementwise_template.cl:14-40, launched by
 * J/backend/main/implementations/elementwise/CLBiElementwise.java:11-24.
 * d < 0: drain = a op b; d = 0/1: partial derivative w.r.t. a / b
 * (J/backend/main/implementations/elementwise/CPUBiElementWise*.java). */
int nk_elementwise(nk_dev dev, int op_id, int d, int dtype, int rank,
                   nk_buf drn, const int32_t* drn_cfg, nk_buf a, const int32_t* a_cfg,
                   nk_buf b, const int32_t* b_cfg, int64_t n);

/* scalarization_<op>_<type>: K/scalarization_template.cl:26-49, launched by
 * J/backend/main/implementations/broadcast/CLScalarBroadcast*.java.  drain = src op value. */
int nk_scalarization(nk_dev dev, int op_id, int d, int dtype, int rank,
                     nk_buf drn, const int32_t* drn_cfg, nk_buf src, const int32_t* src_cfg,
                     double value, int64_t n);

/* scalarization_<op>_<type> for type in {int, long, short, char}: the integer kernels that
 * J/backend/main/implementations/broadcast/CLScalarBroadcast.java:40-58 generates beside float and double.
 * dtype is one of NK_I32, NK_I64, NK_I16, NK_I8; value is narrowed to it (Number.intValue() ...).  The arithmetic
 * is the CPU device's: J/backend/main/implementations/broadcast/CPUScalarBroadcast.java:83-190 with the operator
 * classes beside it and the defaults of J/backend/main/implementations/fun/api/CPUBiFun.java:9-27 -- int and long
 * wrap and truncate like Java, short and byte are evaluated in double and narrowed with Math.round.  A zero
 * divisor of a forward int or long division or modulo is an argument error ("/ by zero", the CPU device's
 * ArithmeticException).  d < 0: drain = src op value; d = 0 / 1: derivative by the element / by the value. */
int nk_scalarization_int(nk_dev dev, int op_id, int d, int dtype, int rank,
                         nk_buf drn, const int32_t* drn_cfg, nk_buf src, const int32_t* src_cfg,
                         int64_t value, int64_t n);

/* scalar_broadcast: K/scalar_broadcast.cl:12-23, launched by
 * J/backend/main/algorithms/ScalarBroadcast.java:65-81.  drain[i] = value through the drain's view. */
int nk_scalar_fill(nk_dev dev, int dtype, int rank, nk_buf drn, const int32_t* drn_cfg, double value, int64_t n);

/* broadcast_<op>: K/broadcast_template.cl:21-113, launched by
 * J/backend/main/implementations/broadcast/CLBroadcast.java:12-24.
 * d < 0: forward broadcast; d >= 0: reducing backward.  CPU semantics:
 * J/backend/main/implementations/broadcast/CPUBroadcast.java:163-259. */
int nk_broadcast(nk_dev dev, int op_id, int d, int dtype, int rank,
                 nk_buf drn, const int32_t* drn_cfg, nk_buf a, const int32_t* a_cfg,
                 nk_buf b, const int32_t* b_cfg, int64_t n);

/* convolution_<op>: K/convolution_template.cl:11-142, launched by
 * J/backend/main/implementations/convolution/CLConvolution.java:11-23.
 * d < 0: nd cross-correlation (drain, src1, src2); d >= 0: gradient ("deconvolution") with the slots
 * as ConvUtil.executeRecursively delivers them (drain = zeros like the gradient target,
 * src1 = the other operand, src2 = error).  CPU semantics (the parity target, not the OpenCL twin):
 * J/backend/main/implementations/convolution/AbstractCPUConvolution.java:245-408. */
int nk_convolution(nk_dev dev, int d, int dtype, int rank,
                   nk_buf drn, const int32_t* drn_cfg, nk_buf a, const int32_t* a_cfg,
                   nk_buf b, const int32_t* b_cfg, int64_t n);

/* fast_local_mem_based_sum / fast_private_sum_reduction: J/backend/main/operations/linear/internal/opencl/CLSum.java:24-62.
 * out[0] = sum of the n elements of the dense buffer `in` (16-byte aligned), reduced in the CPU device's tree --
 * tiles of 128 front to back, recursively (J/backend/main/operations/other/internal/CPUSum.java:26-74) -- so the
 * result is bit-identical to the CPU device's. */
int nk_sum(nk_dev dev, int dtype, nk_buf in, int64_t n, nk_buf out);

/* nk_sum for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  No counterpart in the reference.  Same result as nk_sum, bit for bit; the partial results
 * of the tree live in a 1 MiB array that is part of the library's device image (one copy per GPU, held until the
 * process ends) instead of the grow-on-demand device workspace, so the call neither allocates nor frees.
 * n <= NK_SUM_STATIC_MAX_N, larger inputs are an argument error.  Calls that overlap in time on one GPU share the
 * array and race; nothing in it has to be cleared between calls (every slot is written before it is read). */
#define NK_SUM_STATIC_MAX_N ((int64_t)1 << 30)
int nk_sum_static(nk_dev dev, int dtype, nk_buf in, int64_t n, nk_buf out);

/* CLReduce (min / max): J/backend/main/operations/linear/internal/opencl/CLReduce.java, registered in
 * J/backend/main/operations/other/Min.java:72-73 and Max.java:72-73.  Writes to out_index[0] (int32) the index of
 * the minimum or maximum of the n elements of `in`, found as the CPU device finds it: tiles of 64, strict
 * comparison, first winner stays (J/backend/main/operations/other/internal/CPUReduce.java:90-157). */
enum { NK_REDUCE_MIN = 0, NK_REDUCE_MAX = 1 };
int nk_reduce_index(nk_dev dev, int kind, int dtype, nk_buf in, int64_t n, nk_buf out_index);

/* multiply_arrays_for_dot_product + CLSum: J/backend/main/implementations/linear/CLDot.java:20-56.
 * out[0] = sum of a[i] * b[i]: rounded products, summed in the tree of nk_sum (the CPU device's
 * DOT.unrolled04 keeps four serial running sums; results agree within the reduction tolerance). */
int nk_dot(nk_dev dev, int dtype, nk_buf a, nk_buf b, int64_t n, nk_buf out);

/* simple_matMul / fast_CM_MM_*: J/backend/main/implementations/matmul/CLMatMul.java:11-53,
 * J/backend/main/operations/linear/internal/opencl/CLGEMM.java:11-100.
 * C[M,N] += A[M,K] @ B[K,N] on dense matrices of one layout; C is accumulated into, as the reference
 * does (J/backend/main/operations/linear/internal/blas/GEMM.java:282-304; C is pre-zeroed by
 * J/backend/main/algorithms/MatMulAlgorithm.java:74-85).
 * Below 2^24 multiply-adds, and for an inner dimension of at most 16 (with more than 16 columns), every element is
 * the reference's own sum, term by term in k order with rounded products: bit-identical to the CPU device.  From
 * 2^24 multiply-adds on the sum is re-ordered (matrix cores, or fused multiply-adds in the plans for a few rows or
 * columns) and agrees within 1e-5 (f32) / 1e-12 (f64) of sum_k |a_ik| |b_kj|; WHICH plan runs depends on the shape
 * and on whether A, B and C start on 16-byte boundaries, so the same product taken from a view at an odd offset may
 * differ in its last bits from the one taken from the start of a buffer. */
int nk_matmul(nk_dev dev, int dtype, int layout, int64_t M, int64_t K, int64_t N,
              nk_buf A, nk_buf B, nk_buf C);

/* simple_matMul as the OpenCL device runs it: J/backend/main/implementations/matmul/CLMatMul.java:35-52, whose kernel
 * ends in `C[ n + m * N ] = acc` (:50).  C[M,N] = A[M,K] @ B[K,N]: the old contents of C are neither read nor
 * kept, which saves their trip from memory (a third of the traffic of a product with a short inner dimension).
 * On a zeroed C -- the only way the reference calls either (MatMulAlgorithm.java:74-85) -- the result equals nk_matmul's
 * bit for bit.  Same arguments, limits and errors as nk_matmul. */
int nk_matmul_set(nk_dev dev, int dtype, int layout, int64_t M, int64_t K, int64_t N,
                  nk_buf A, nk_buf B, nk_buf C);

/* Fused elementwise expression, the device side of Device.optimizedFunctionOf
 * (J/devices/Device.java:216-243; J/devices/opencl/utility/CLFunctionCompiler.java:101-199).
 * `program` is a postfix op-code sequence of `n_ops` int32 words evaluated per drain element on a
 * small value stack:
 *     NK_FUSE_LOAD  k   push source k (0 <= k < n_src)
 *     NK_FUSE_CONST k   push consts[k]
 *     NK_FUSE_FUN   id  replace the top of the stack with fun id applied to it (NK_FUN_*)
 *     NK_FUSE_DFUN  id  same with the derivative of fun id
 *     NK_FUSE_BIN   op  pop b, pop a, push a op b (NK_OP_ADD..NK_OP_POW)
 * The single value left on the stack is stored to the drain.  Each intermediate is rounded to the
 * tensor dtype exactly as the unfused kernels round it, so + - * stay bit-identical to the unfused
 * sequence.  n_src <= NK_FUSE_MAX_SRC, n_ops <= NK_FUSE_MAX_OPS, stack depth <= NK_FUSE_MAX_STACK per launch, and at most
 * NK_FUSE_MAX_SAVED computed operands may wait at once for the evaluation of their right-hand neighbour (a plain source
 * or constant never waits: it is read where it is used).  The host cuts a larger expression into several launches
 * through temporaries, which changes no result because of that rounding. */
enum { NK_FUSE_LOAD = 0, NK_FUSE_CONST = 1, NK_FUSE_FUN = 2, NK_FUSE_DFUN = 3, NK_FUSE_BIN = 4 };
#define NK_FUSE_MAX_SRC 6
#define NK_FUSE_MAX_OPS 32
#define NK_FUSE_MAX_STACK 8
#define NK_FUSE_MAX_CONST 8
#define NK_FUSE_MAX_SAVED 4
int nk_fused(nk_dev dev, const int32_t* program, int n_ops, const double* consts, int n_consts,
             int dtype, int rank, nk_buf drn, const int32_t* drn_cfg,
             int n_src, const nk_buf* srcs, const int32_t* const* src_cfgs, int64_t n);

#ifdef __cplusplus
}
#endif
#endif /* NEUREKA_HIP_H */
