package neureka.devices.hip;

import neureka.Tensor;

import java.lang.foreign.*;
import java.lang.invoke.MethodHandle;
import static java.lang.foreign.ValueLayout.*;

/** Downcalls into libneureka_hip.so.  I = int, J = long (nk_dev, nk_buf, sizes, events), D = double, P = pointer. */
public final class Nk {
    private static final Linker L = Linker.nativeLinker();
    private static final SymbolLookup LIB =
        SymbolLookup.libraryLookup(System.getProperty("neureka.hip.lib", "libneureka_hip.so"), Arena.global());
    private static final ValueLayout I = JAVA_INT, J = JAVA_LONG, D = JAVA_DOUBLE, P = ADDRESS;
    private static MethodHandle h(String name, MemoryLayout res, MemoryLayout... args) {
        return L.downcallHandle(LIB.find(name).orElseThrow(() -> new UnsatisfiedLinkError(name)), FunctionDescriptor.of(res, args));
    }

    // diagnostics
    public static final MethodHandle nk_last_error        = h("nk_last_error", P);
    public static final MethodHandle nk_last_path         = h("nk_last_path", P);
    // lifecycle
    public static final MethodHandle nk_device_count      = h("nk_device_count", I, P);
    public static final MethodHandle nk_device_open       = h("nk_device_open", I, I, P);
    public static final MethodHandle nk_device_close      = h("nk_device_close", I, J);
    public static final MethodHandle nk_device_sync       = h("nk_device_sync", I, J);
    public static final MethodHandle nk_device_props      = h("nk_device_props", I, J, P, J, P, P, P, P, P);
    public static final MethodHandle nk_device_memory     = h("nk_device_memory", I, J, P, P);
    public static final MethodHandle nk_device_stats      = h("nk_device_stats", I, J, P, P);
    // memory: nk_alloc hands out a block of the pool with arbitrary contents, nk_free gives it back without a wait
    public static final MethodHandle nk_alloc             = h("nk_alloc", I, J, J, P);
    public static final MethodHandle nk_free              = h("nk_free", I, J, J);
    public static final MethodHandle nk_pool_trim         = h("nk_pool_trim", I, J);
    public static final MethodHandle nk_pool_stats        = h("nk_pool_stats", I, J, P, P, P, P);
    public static final MethodHandle nk_pool_config       = h("nk_pool_config", I, J, J, I);
    public static final MethodHandle nk_h2d               = h("nk_h2d", I, J, J, J, P, J);
    public static final MethodHandle nk_d2h               = h("nk_d2h", I, J, P, J, J, J);
    public static final MethodHandle nk_d2d               = h("nk_d2d", I, J, J, J, J, J, J);
    public static final MethodHandle nk_fill              = h("nk_fill", I, J, J, J, P, I, J);
    // timing
    public static final MethodHandle nk_event_create      = h("nk_event_create", I, J, P);
    public static final MethodHandle nk_event_record      = h("nk_event_record", I, J, J);
    public static final MethodHandle nk_event_elapsed_ms  = h("nk_event_elapsed_ms", I, J, J, J, P);
    public static final MethodHandle nk_event_destroy     = h("nk_event_destroy", I, J, J);
    // kernels: (dev, id, d, dtype, rank, drain, drain cfg, sources with their cfgs ..., n)
    public static final MethodHandle nk_activation        = h("nk_activation", I, J, I, I, I, I, J, P, J, P, J);
    public static final MethodHandle nk_elementwise       = h("nk_elementwise", I, J, I, I, I, I, J, P, J, P, J, P, J);
    public static final MethodHandle nk_scalarization     = h("nk_scalarization", I, J, I, I, I, I, J, P, J, P, D, J);
    public static final MethodHandle nk_scalarization_int = h("nk_scalarization_int", I, J, I, I, I, I, J, P, J, P, J, J);
    public static final MethodHandle nk_scalar_fill       = h("nk_scalar_fill", I, J, I, I, J, P, D, J);
    public static final MethodHandle nk_broadcast         = h("nk_broadcast", I, J, I, I, I, I, J, P, J, P, J, P, J);
    public static final MethodHandle nk_convolution       = h("nk_convolution", I, J, I, I, I, J, P, J, P, J, P, J);
    public static final MethodHandle nk_matmul            = h("nk_matmul", I, J, I, I, J, J, J, J, J, J);
    public static final MethodHandle nk_matmul_set        = h("nk_matmul_set", I, J, I, I, J, J, J, J, J, J);
    public static final MethodHandle nk_sum               = h("nk_sum", I, J, I, J, J, J);
    public static final MethodHandle nk_sum_static        = h("nk_sum_static", I, J, I, J, J, J);
    public static final MethodHandle nk_reduce_index      = h("nk_reduce_index", I, J, I, I, J, J, J);
    public static final MethodHandle nk_dot               = h("nk_dot", I, J, I, J, J, J, J);
    public static final MethodHandle nk_fused             = h("nk_fused", I, J, P, I, P, I, I, I, J, P, I, P, P, J);

    /** Runs a downcall that returns a status; a non-zero status becomes the exception the caller expects. */
    public interface Call { int run() throws Throwable; }
    public static void check(Call c) {
        int status;
        try { status = c.run(); } catch (RuntimeException | Error e) { throw e; } catch (Throwable t) { throw new AssertionError(t); }
        if (status != 0) throw new IllegalStateException("[" + status + "] " + lastError());
    }
    public static String lastError() {
        try { return ((MemorySegment) nk_last_error.invokeExact()).reinterpret(1024).getString(0); }
        catch (Throwable t) { throw new AssertionError(t); }
    }
    /** NDConfiguration.asInlineArray() as a native int32 array that lives as long as the arena. */
    public static MemorySegment cfg(Arena a, Tensor<?> t) {
        int[] inline = t.isVirtual() ? new int[5 * t.rank()] : t.getNDConf().asInlineArray();
        if (t.isVirtual()) System.arraycopy(t.getNDConf().shape(), 0, inline, 0, t.rank());   // all-zero tables, shape kept
        return a.allocateFrom(JAVA_INT, inline);
    }
}
