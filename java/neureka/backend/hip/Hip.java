package neureka.backend.hip;

import neureka.Shape;
import neureka.Tensor;
import neureka.backend.api.ExecutionCall;
import neureka.backend.main.implementations.fun.api.CPUFun;
import neureka.backend.main.implementations.fun.api.ScalarFun;
import neureka.devices.hip.HipDevice;
import neureka.devices.hip.Nk;
import neureka.math.args.Arg;
import neureka.ndim.config.NDConfiguration;

import java.lang.foreign.Arena;
import java.lang.foreign.MemorySegment;
import java.lang.invoke.MethodHandle;
import java.util.Arrays;
import java.util.List;
import static java.lang.foreign.ValueLayout.*;

/** The ImplementationFor<HipDevice> bodies: one downcall each, slots in the reference's order (drain first). */
public final class Hip {
    private static int d(ExecutionCall<HipDevice> c) { return c.getValOf(Arg.DerivIdx.class); }
    /** NK_FUN_* = position in this list: the ids of ScalarFun.java:7-31 in the order of include/neureka_hip.h */
    public static final List<String> FUN_IDS = Arrays.asList("abs", "cos", "gasu", "gatu", "gaus", "fast_gaus", "gelu", "idy", "ln", "quad", "relu", "selu",
                                                             "sig", "silu", "sin", "softplus", "softsign", "tanh", "fast_tanh", "exp", "log10", "sqrt", "cbrt");
    /** NK_OP_* = position in this list: the identifiers of the six operators */
    public static final List<String> OP_IDS = Arrays.asList("add", "subtract", "multiply", "divide", "modulo", "power");
    private static int funId(ScalarFun f) { return FUN_IDS.indexOf(f.id()); }
    private static boolean integral(Tensor<?> t) { Class<?> c = t.itemType(); return c == Integer.class || c == Long.class || c == Short.class || c == Byte.class; }

    static Tensor<?> activation(ScalarFun f, ExecutionCall<HipDevice> c) {     // CLElementwiseFunction.java:27-41
        Tensor<?> drn = c.input(0), src = c.input(1); long dev = c.getDevice().handle;
        try (Arena a = Arena.ofConfined()) {
            MemorySegment c0 = Nk.cfg(a, drn), c1 = Nk.cfg(a, src);
            Nk.check(() -> (int) Nk.nk_activation.invokeExact(dev, funId(f), d(c), HipDevice.dtype(drn.itemType()), drn.rank(),
                                                             HipDevice.ptr(drn), c0, HipDevice.ptr(src), c1, (long) drn.size()));
        }
        return drn;
    }
    static Tensor<?> elementwise(int op, ExecutionCall<HipDevice> c) { return binary(Nk.nk_elementwise, op, c); }   // CLBiElementwise.java:11-24
    static Tensor<?> broadcast(int op, ExecutionCall<HipDevice> c)   { return binary(Nk.nk_broadcast, op, c); }     // CLBroadcast.java:12-24
    private static Tensor<?> binary(MethodHandle entry, int op, ExecutionCall<HipDevice> c) {
        Tensor<?> drn = c.input(0), x = c.input(1), y = c.input(2); long dev = c.getDevice().handle;
        try (Arena a = Arena.ofConfined()) {
            MemorySegment c0 = Nk.cfg(a, drn), c1 = Nk.cfg(a, x), c2 = Nk.cfg(a, y);
            Nk.check(() -> (int) entry.invokeExact(dev, op, d(c), HipDevice.dtype(drn.itemType()), drn.rank(),
                                                   HipDevice.ptr(drn), c0, HipDevice.ptr(x), c1, HipDevice.ptr(y), c2, (long) drn.size()));
        }
        return drn;
    }
    static Tensor<?> scalarization(int op, ExecutionCall<HipDevice> c) {       // CLScalarBroadcastAddition.java:15-34 and its siblings
        Tensor<?> drn = c.input(0), src = c.input(1); Number v = c.input(Number.class, 2).at(0).get();
        return scalarization(op, c, drn, src, v);
    }
    static Tensor<?> scalarizationIdentity(ExecutionCall<HipDevice> c) {       // CLScalarBroadcastIdentity.java:18-32
        Tensor<?> drn = c.input(0); Number v = c.input(Number.class, 1).at(0).get();
        return scalarization(6 /* NK_OP_IDY */, c, drn, drn, v);
    }
    private static Tensor<?> scalarization(int op, ExecutionCall<HipDevice> c, Tensor<?> drn, Tensor<?> src, Number v) {
        long dev = c.getDevice().handle;
        try (Arena a = Arena.ofConfined()) {
            MemorySegment c0 = Nk.cfg(a, drn), c1 = Nk.cfg(a, src);
            if (integral(drn))
                Nk.check(() -> (int) Nk.nk_scalarization_int.invokeExact(dev, op, d(c), HipDevice.dtype(drn.itemType()), drn.rank(),
                                                                        HipDevice.ptr(drn), c0, HipDevice.ptr(src), c1, v.longValue(), (long) drn.size()));
            else
                Nk.check(() -> (int) Nk.nk_scalarization.invokeExact(dev, op, d(c), HipDevice.dtype(drn.itemType()), drn.rank(),
                                                                    HipDevice.ptr(drn), c0, HipDevice.ptr(src), c1, v.doubleValue(), (long) drn.size()));
        }
        return drn;
    }
    static Tensor<?> scalarFunction(ScalarFun f, ExecutionCall<HipDevice> c) { // CLScalarFunction.java:20-28: host f, one item written
        CPUFun g = d(c) < 0 ? f.getActivation() : f.getDerivative();
        Number value = g.invoke(c.input(Number.class, 1).item(0).doubleValue());
        c.input(Number.class, 0).mut().setDataAt(0, value);                   // -> HipDevice._writeItem -> nk_fill
        return c.input(0);
        // (the Python mirror runs nk_activation on the one stored element instead: no host round trip, same contract)
    }
    static Tensor<?> scalarBroadcast(ScalarFun f, ExecutionCall<HipDevice> c) { // ScalarBroadcast.java:64-81
        CPUFun g = d(c) < 0 ? f.getActivation() : f.getDerivative();
        double value = g.invoke(c.input(Number.class, 1).at(0).get().doubleValue());
        Tensor<Number> t = c.input(Number.class, 0); long dev = c.getDevice().handle;
        try (Arena a = Arena.ofConfined()) {
            MemorySegment c0 = Nk.cfg(a, t);
            Nk.check(() -> (int) Nk.nk_scalar_fill.invokeExact(dev, HipDevice.dtype(t.itemType()), t.rank(), HipDevice.ptr(t), c0, value, (long) t.size()));
        }
        return t;
    }
    static Tensor<?> convolution(ExecutionCall<HipDevice> c) {                 // CLConvolution.java:11-23
        Tensor<?> drn = c.input(0), x = c.input(1), y = c.input(2); long dev = c.getDevice().handle;
        try (Arena a = Arena.ofConfined()) {
            MemorySegment c0 = Nk.cfg(a, drn), c1 = Nk.cfg(a, x), c2 = Nk.cfg(a, y);
            Nk.check(() -> (int) Nk.nk_convolution.invokeExact(dev, c.getDerivativeIndex(), HipDevice.dtype(drn.itemType()), drn.rank(),
                                                              HipDevice.ptr(drn), c0, HipDevice.ptr(x), c1, HipDevice.ptr(y), c2, (long) drn.size()));
        }
        return drn;
    }
    static Tensor<?> matMul(ExecutionCall<HipDevice> c) {                      // CLMatMul.java:11-53 with the layout checks of CPUMatMul.java:17-96
        Tensor<?> C = c.input(0), A = c.input(1), B = c.input(2);
        boolean rowMajor = A.getNDConf().getLayout() != NDConfiguration.Layout.COLUMN_MAJOR && B.getNDConf().getLayout() != NDConfiguration.Layout.COLUMN_MAJOR;
        long M = A.shape(0), K = A.shape(1), N = B.shape(1), dev = c.getDevice().handle;
        // C = A @ B like simple_matMul (CLMatMul.java:50); the drain arrives zeroed (MatMulAlgorithm.java:74-85), so nk_matmul gives the same bits
        Nk.check(() -> (int) Nk.nk_matmul_set.invokeExact(dev, HipDevice.dtype(C.itemType()), rowMajor ? 0 : 1, M, K, N,
                                                         HipDevice.ptr(A), HipDevice.ptr(B), HipDevice.ptr(C)));
        return C;
    }
    static Tensor<?> sum(ExecutionCall<HipDevice> c) {                         // CLSum.java:24-62
        Tensor<?> in = c.input(0); HipDevice dev = c.getDevice();
        Tensor<?> out = Tensor.of(in.itemType(), Shape.of(1), 0).mut().setIsVirtual(false).to(dev);
        Nk.check(() -> (int) Nk.nk_sum.invokeExact(dev.handle, HipDevice.dtype(in.itemType()), HipDevice.ptr(in), (long) in.size(), HipDevice.ptr(out)));
        return out;                                                           // nk_sum_static: same arguments, never allocates, n <= 2^30
    }
    static Tensor<?> dot(ExecutionCall<HipDevice> c) {                         // CLDot.java:20-56
        Tensor<?> x = c.input(0), y = c.input(1); HipDevice dev = c.getDevice();
        Tensor<?> out = Tensor.of(x.itemType(), Shape.of(1), 0).mut().setIsVirtual(false).to(dev);
        Nk.check(() -> (int) Nk.nk_dot.invokeExact(dev.handle, HipDevice.dtype(x.itemType()), HipDevice.ptr(x), HipDevice.ptr(y), (long) x.size(), HipDevice.ptr(out)));
        return out;
    }
    static Tensor<?> reduce(int kind, ExecutionCall<HipDevice> c) {            // CLReduce + Min.java:43-52
        Tensor<?> in = c.input(0); HipDevice dev = c.getDevice();
        Tensor<Integer> index = Tensor.of(Integer.class, Shape.of(1), 0).mut().setIsVirtual(false).to(dev);
        Nk.check(() -> (int) Nk.nk_reduce_index.invokeExact(dev.handle, kind, HipDevice.dtype(in.itemType()), HipDevice.ptr(in), (long) in.size(), HipDevice.ptr(index)));
        return index;                                                         // Min.java reads index.item(0) and wraps in.item(i)
    }
    /** One launch of nk_fused: program / consts as HipFunctionCompiler lowers them (CLFunctionCompiler.java:101-199). */
    public static Tensor<?> fused(HipDevice dev, int[] program, double[] consts, Tensor<?> drn, Tensor<?>[] srcs) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment prog = a.allocateFrom(JAVA_INT, program), cs = a.allocateFrom(JAVA_DOUBLE, consts.length == 0 ? new double[1] : consts);
            MemorySegment ptrs = a.allocate(JAVA_LONG, srcs.length), cfgs = a.allocate(ADDRESS, srcs.length), c0 = Nk.cfg(a, drn);
            for (int i = 0; i < srcs.length; i++) { ptrs.setAtIndex(JAVA_LONG, i, HipDevice.ptr(srcs[i])); cfgs.setAtIndex(ADDRESS, i, Nk.cfg(a, srcs[i])); }
            Nk.check(() -> (int) Nk.nk_fused.invokeExact(dev.handle, prog, program.length / 2, cs, consts.length, HipDevice.dtype(drn.itemType()), drn.rank(),
                                                         HipDevice.ptr(drn), c0, srcs.length, ptrs, cfgs, (long) drn.size()));
        }
        return drn;
    }
    // timing helpers for benchmarks: nk_event_create / nk_event_record / nk_event_elapsed_ms / nk_event_destroy bracket launches on the device's
    // own stream; nk_d2d copies between buffers on it; nk_device_stats backs leak tests (numberOfDataObjects); nk_last_path names the kernel taken
}
