package neureka.backend.hip;

import neureka.Neureka;
import neureka.backend.api.BackendContext;
import neureka.backend.api.BackendExtension;
import neureka.backend.api.DeviceAlgorithm;
import neureka.backend.api.Extensions;
import neureka.backend.api.Operation;
import neureka.backend.api.ini.BackendLoader;
import neureka.backend.api.ini.ReceiveForDevice;
import neureka.backend.main.algorithms.*;
import neureka.backend.main.implementations.fun.api.ScalarFun;
import neureka.backend.main.operations.functions.*;
import neureka.backend.main.operations.linear.*;
import neureka.backend.main.operations.operator.*;
import neureka.backend.main.operations.other.AssignLeft;
import neureka.backend.main.operations.other.Randomization;
import neureka.backend.main.operations.other.Sum;
import neureka.devices.hip.HipDevice;
import neureka.devices.hip.Nk;

import java.lang.foreign.Arena;
import java.lang.foreign.MemorySegment;
import java.util.ArrayList;
import java.util.Arrays;
import java.util.LinkedHashMap;
import java.util.List;
import java.util.Map;
import static java.lang.foreign.ValueLayout.JAVA_INT;

/** Model: neureka.backend.ocl.CLBackend (find: :56-94, update: :96-152, _load: :200-325). */
public final class HipBackend implements BackendExtension {
    private final List<HipDevice> devices = new ArrayList<>();
    @Override public boolean update(OwnerChangeRequest<Extensions> r) {     // opens the devices when the extension is installed
        if (r.type() == IsBeing.ADDED && devices.isEmpty()) try (Arena a = Arena.ofConfined()) {
            MemorySegment n = a.allocate(JAVA_INT);
            Nk.check(() -> (int) Nk.nk_device_count.invokeExact(n));
            for (int i = 0; i < n.get(JAVA_INT, 0); i++) devices.add(new HipDevice(i));
        }
        r.executeChange(); return true;
    }
    @Override public DeviceOption find(String key) {                        // keyword confidence like CLBackend.find
        if (devices.isEmpty()) return new DeviceOption(null, 0);
        String k = key.toLowerCase().trim();
        for (String w : new String[]{"hip", "rocm", "amd", "radeon", "gpu", "first gpu", "mi355x", "instinct"})
            if (k.equals(w) || Arrays.asList(k.split(" ")).contains(w)) return new DeviceOption(devices.get(0), 1.0);
        for (HipDevice d : devices) if (d.name().toLowerCase().contains(k)) return new DeviceOption(d, 1.0);
        return new DeviceOption(devices.get(0), 0);
    }
    @Override public void reset() {}
    @Override public void dispose() { devices.forEach(HipDevice::dispose); devices.clear(); }
    @Override public BackendLoader getLoader() { return registry -> _load(registry.forDevice(HipDevice.class)); }

    private void _load(ReceiveForDevice<HipDevice> r) {
        // the six operators: three rows each (CLBackend.java:202-230)
        Map<Class<? extends Operation>, Integer> ops = Map.of(Addition.class, 0, Subtraction.class, 1, Multiplication.class, 2,
                                                              Division.class, 3, Modulo.class, 4, Power.class, 5);       // NK_OP_*
        ops.forEach((type, op) -> r.forOperation(type)
            .set(BiScalarBroadcast.class, ctx -> call -> Hip.scalarization(op, call))      // nk_scalarization / nk_scalarization_int
            .set(Broadcast.class,         ctx -> call -> Hip.broadcast(op, call))          // nk_broadcast
            .set(BiElementwise.class,     ctx -> call -> Hip.elementwise(op, call)));      // nk_elementwise
        // AssignLeft (CLBackend.java:232-234)
        r.forOperation(AssignLeft.class)
            .set(BiScalarBroadcast.class,    ctx -> call -> Hip.scalarizationIdentity(call))          // nk_scalarization(NK_OP_IDY): drain passed as drain and source
            .set(ElementwiseAlgorithm.class, ctx -> call -> Hip.activation(ScalarFun.IDENTITY, call)); // nk_activation(NK_FUN_IDY)
        // convolution (CLBackend.java:236-241): nk_convolution, d = call.getDerivativeIndex()
        r.forOperation(Convolution.class).set(NDConvolution.class, ctx -> Hip::convolution);
        r.forOperation(XConvLeft.class)  .set(NDConvolution.class, ctx -> Hip::convolution);
        r.forOperation(XConvRight.class) .set(NDConvolution.class, ctx -> Hip::convolution);
        r.forOperation(MatMul.class)     .set(MatMulAlgorithm.class,     ctx -> Hip::matMul);   // nk_matmul_set  (CLBackend.java:243-244)
        r.forOperation(DotProduct.class) .set(DotProductAlgorithm.class, ctx -> Hip::dot);      // nk_dot     (:246-247)
        r.forOperation(Sum.class)        .set(SumAlgorithm.class,        ctx -> Hip::sum);      // nk_sum     (:249-250)
        r.forOperation(Randomization.class).set(ElementwiseAlgorithm.class,                     // (:252-253) CLRandomization is a stub that throws
            ctx -> call -> { throw new IllegalStateException("Not yet implemented"); });
        // the 23 activations: ElementwiseAlgorithm + ScalarAlgorithm each (CLBackend.java:255-324)
        Map<Class<? extends Operation>, ScalarFun> funs = new LinkedHashMap<>();
        funs.put(Absolute.class, ScalarFun.ABSOLUTE);   funs.put(Cosinus.class, ScalarFun.COSINUS);     funs.put(GaSU.class, ScalarFun.GASU);
        funs.put(GaTU.class, ScalarFun.GATU);           funs.put(Gaussian.class, ScalarFun.GAUSSIAN);   funs.put(GaussianFast.class, ScalarFun.GAUSSIAN_FAST);
        funs.put(GeLU.class, ScalarFun.GELU);           funs.put(Identity.class, ScalarFun.IDENTITY);   funs.put(Logarithm.class, ScalarFun.LOGARITHM);
        funs.put(Quadratic.class, ScalarFun.QUADRATIC); funs.put(ReLU.class, ScalarFun.RELU);           funs.put(SeLU.class, ScalarFun.SELU);
        funs.put(Sigmoid.class, ScalarFun.SIGMOID);     funs.put(SiLU.class, ScalarFun.SILU);           funs.put(Sinus.class, ScalarFun.SINUS);
        funs.put(Softplus.class, ScalarFun.SOFTPLUS);   funs.put(Softsign.class, ScalarFun.SOFTSIGN);   funs.put(Tanh.class, ScalarFun.TANH);
        funs.put(TanhFast.class, ScalarFun.TANH_FAST);  funs.put(Exp.class, ScalarFun.EXP);             funs.put(Cbrt.class, ScalarFun.CBRT);
        funs.put(Log10.class, ScalarFun.LOG10);         funs.put(Sqrt.class, ScalarFun.SQRT);
        funs.forEach((type, fun) -> r.forOperation(type)
            .set(ElementwiseAlgorithm.class, ctx -> call -> Hip.activation(fun, call))          // nk_activation
            .set(ScalarAlgorithm.class,      ctx -> call -> Hip.scalarFunction(fun, call)));     // CLScalarFunction.java:20-28
        // ScalarBroadcast registers its OpenCL implementation in its own constructor (ScalarBroadcast.java:64-82), and
        // Min / Max theirs on the algorithm (Min.java:72-73): the HIP implementations are attached the same way
        BackendContext backend = Neureka.get().backend();
        funs.forEach((type, fun) -> backend.getOperation(fun.id()).getAlgorithm(ScalarBroadcast.class)
            .setImplementationFor(HipDevice.class, call -> Hip.scalarBroadcast(fun, call)));     // nk_scalar_fill
        backend.getOperation("min").getAlgorithm(DeviceAlgorithm.class).setImplementationFor(HipDevice.class, call -> Hip.reduce(0, call));   // nk_reduce_index
        backend.getOperation("max").getAlgorithm(DeviceAlgorithm.class).setImplementationFor(HipDevice.class, call -> Hip.reduce(1, call));
    }
}
