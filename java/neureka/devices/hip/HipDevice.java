package neureka.devices.hip;

import neureka.Data;
import neureka.Tensor;
import neureka.backend.api.ExecutionCall;
import neureka.backend.api.Operation;
import neureka.common.composition.Component;
import neureka.common.utility.DataConverter;
import neureka.devices.AbstractDevice;
import neureka.devices.AbstractDeviceData;
import neureka.devices.Device;
import neureka.dtype.DataType;
import neureka.framing.Relation;
import neureka.math.Function;
import neureka.ndim.NDConstructor;
import neureka.ndim.config.NDConfiguration;

import java.lang.foreign.Arena;
import java.lang.foreign.MemorySegment;
import static java.lang.foreign.ValueLayout.*;

/** Model: neureka.devices.opencl.OpenCLDevice (store/restore/free, CLData ownership, virtual tensors). */
public final class HipDevice extends AbstractDevice<Number> {
    public final long handle;                            // nk_dev
    private final String name; private final int computeUnits, clockMHz, ldsBytes, wavefront; private final long globalMem;

    public HipDevice(int index) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment out = a.allocate(JAVA_LONG);
            Nk.check(() -> (int) Nk.nk_device_open.invokeExact(index, out));
            handle = out.get(JAVA_LONG, 0);
            MemorySegment nm = a.allocate(256), cu = a.allocate(JAVA_INT), mhz = a.allocate(JAVA_INT), mem = a.allocate(JAVA_LONG),
                          lds = a.allocate(JAVA_INT), wave = a.allocate(JAVA_INT);
            Nk.check(() -> (int) Nk.nk_device_props.invokeExact(handle, nm, 256L, cu, mhz, mem, lds, wave));
            name = nm.getString(0); computeUnits = cu.get(JAVA_INT, 0); clockMHz = mhz.get(JAVA_INT, 0);
            globalMem = mem.get(JAVA_LONG, 0); ldsBytes = lds.get(JAVA_INT, 0); wavefront = wave.get(JAVA_INT, 0);
        }
    }

    /** A device buffer; freed by nk_free when its usage count reaches 0 or when it becomes phantom reachable
     *  (AbstractDeviceData registers the action with the DeviceCleaner): OpenCLDevice.java:950-966. */
    static final class HipData extends AbstractDeviceData<Number> {
        final long ptr; final int length;                // nk_buf, elements
        HipData(HipDevice owner, long ptr, int length, DataType<Number> type) {
            super(owner, ptr, type, () -> Nk.check(() -> (int) Nk.nk_free.invokeExact(owner.handle, ptr)));
            this.ptr = ptr; this.length = length;
        }
    }
    public static long ptr(Tensor<?> t) { return ((HipData) t.getMut().getData()).ptr; }
    public static int dtype(Class<?> c) {                       // NK_F32 ... NK_I8
        if (c == Float.class) return 0;  if (c == Double.class) return 1; if (c == Integer.class) return 2;
        if (c == Long.class) return 3;   if (c == Short.class) return 4;  if (c == Byte.class) return 5;
        throw new IllegalArgumentException("HipDevice does not hold items of type " + c.getSimpleName());
    }
    public static int bytes(Class<?> c) { return c == Double.class || c == Long.class ? 8 : c == Short.class ? 2 : c == Byte.class ? 1 : 4; }

    // ---- Device ------------------------------------------------------------------------------------------------
    @Override public void dispose() {                                        // OpenCLDevice.java:299-304
        _numberOfTensors = 0;
        Nk.check(() -> (int) Nk.nk_device_close.invokeExact(handle));     // syncs the stream, frees every live buffer
    }
    @Override public Device<Number> restore(Tensor<Number> t) {              // OpenCLDevice.java:315-334
        if (!has(t)) throw new IllegalArgumentException("The passed tensor cannot be restored from this HIP device because the tensor is not stored on the device.\n");
        Object host = _readAll(t, true);
        free(t);
        t.find(Tensor.class).ifPresent(this::restore);
        t.getMut().setItems(host);
        return this;
    }
    @Override public <T extends Number> Device<Number> store(Tensor<T> t) { t.set((Component) this); return this; }   // -> update()
    @Override public boolean update(OwnerChangeRequest<Tensor<Number>> changeRequest) {                                // OpenCLDevice.java:340-371
        super.update(changeRequest);
        if (changeRequest.type() == IsBeing.ADDED) {
            Tensor<Number> t = changeRequest.getNewOwner();
            Tensor<Number> root = t.isSlice() || t.isShallowCopy() ? t.get(Relation.class).findRootTensor().orElse(null) : null;
            if (root != null) {                                               // a view shares its root's HipData
                if (!root.isOutsourced()) throw new IllegalStateException("Data parent is not outsourced!");
                _add(t, root.getMut().getData(), changeRequest::executeChange);
            } else _add(t, null, changeRequest::executeChange);
            return true;
        }
        return true;
    }
    private void _add(Tensor<Number> t, Data<Number> parentData, Runnable migration) {                                 // OpenCLDevice.java:361-405
        if (has(t)) return;
        Data<Number> data = parentData;
        if (data == null) {
            if (t.getMut().getData().owner() == this) { migration.run(); return; }
            Object host = t.getMut().getData().getOrNull();               // float[] / double[] / int[] / long[] / short[] / byte[]
            int n = t.isVirtual() ? 1 : java.lang.reflect.Array.getLength(host);
            HipData d = _alloc(t.itemType(), n);
            _h2d(d, 0, host, 0, n);                                       // a virtual tensor uploads its single element
            data = d;
        }
        t.getMut().setData(data);
        migration.run();
    }
    @Override public <T extends Number> Device<Number> free(Tensor<T> t) {   // OpenCLDevice.java:609-620
        if (!has(t)) throw new IllegalArgumentException("tensor is not stored on this device");
        t.getMut().setData(null);                                         // decrements the usage count; nk_free at zero
        t.find(Device.class).ifPresent(d -> t.remove(Device.class));
        return this;
    }
    @Override public <T extends Number> Data<T> allocate(DataType<T> type, NDConfiguration ndc) {                      // OpenCLDevice.java:520-530
        return (Data<T>) _alloc(type.getItemTypeClass(), ndc.size());
    }
    @Override public <T extends Number> Data<T> allocateFromOne(DataType<T> type, NDConfiguration ndc, T initialValue) {
        HipData d = _alloc(type.getItemTypeClass(), ndc.size());
        _fill(d, 0, ndc.size(), initialValue);
        return (Data<T>) d;
    }
    @Override public <T extends Number> Data<T> allocateFromAll(DataType<T> type, NDConfiguration ndc, Object jvmData) {
        HipData d = _alloc(type.getItemTypeClass(), ndc.size());
        _h2d(d, 0, jvmData, 0, ndc.size());
        return (Data<T>) d;
    }
    @Override public Operation optimizedOperationOf(Function f, String name) {                                        // Device.java:216-243
        return new HipFunctionCompiler(this, f, name).optimize();   // the expression (and its derivatives) as nk_fused programs
    }
    @Override public Device<Number> approve(ExecutionCall<? extends Device<?>> call) { return this; }
    public void sync() { Nk.check(() -> (int) Nk.nk_device_sync.invokeExact(handle)); }

    // ---- AbstractDevice's protected contract (AbstractDevice.java:188-206) as OpenCLDevice fills it in (:527-660) ---------------
    @Override protected <T extends Number> int _sizeOccupiedBy(Tensor<T> t) { return ((HipData) t.getMut().getData()).length; }
    @Override protected <T extends Number> Object _readAll(Tensor<T> t, boolean clone) { return _readArray(t, null, 0, _sizeOccupiedBy(t)); }
    @Override protected <T extends Number> T _readItem(Tensor<T> t, int index) {
        return (T) (Number) java.lang.reflect.Array.get(_readArray(t, null, index, 1), 0);
    }
    @Override protected <T extends Number, A> A _readArray(Tensor<T> t, Class<A> arrayType, int start, int size) {
        Class<?> item = t.itemType(); int eb = bytes(item);
        try (Arena a = Arena.ofConfined()) {
            MemorySegment host = a.allocate((long) size * eb, 16);
            Nk.check(() -> (int) Nk.nk_d2h.invokeExact(handle, host, ptr(t), (long) start * eb, (long) size * eb));    // blocking
            Object out = item == Float.class ? host.toArray(JAVA_FLOAT) : item == Double.class ? host.toArray(JAVA_DOUBLE)
                       : item == Integer.class ? host.toArray(JAVA_INT) : item == Long.class ? host.toArray(JAVA_LONG)
                       : item == Short.class ? host.toArray(JAVA_SHORT) : host.toArray(JAVA_BYTE);
            return arrayType == null ? (A) out : DataConverter.get().convert(out, arrayType);
        }
    }
    @Override protected <T extends Number> void _writeItem(Tensor<T> t, T item, int start, int size) {                  // a device fill: OpenCLDevice.java:537-541
        _fill((HipData) t.getMut().getData(), start, size, item);
    }
    @Override protected <T extends Number> void _writeArray(Tensor<T> t, Object array, int offset, int start, int size) { // OpenCLDevice.java:542-552
        _h2d((HipData) t.getMut().getData(), start, array, offset, size);
    }
    @Override protected <T extends Number> void _swap(Tensor<T> former, Tensor<T> replacement) {                        // OpenCLDevice.java:635-640
        replacement.getMut().setData(former.getMut().getData());
    }
    @Override protected Data<Number> _actualize(Tensor<?> t) {                                                          // OpenCLDevice.java:573-593
        Number value = _readItem((Tensor<Number>) t, 0);
        HipData full = _alloc(t.itemType(), t.size());
        _fill(full, 0, t.size(), value);
        return full;
    }
    @Override protected Data<Number> _virtualize(Tensor<?> t) {
        Number value = _readItem((Tensor<Number>) t, t.getNDConf().indexOfIndex(0));
        HipData one = _alloc(t.itemType(), 1);
        _fill(one, 0, 1, value);
        return one;
    }
    @Override protected DataType<?> _dataTypeOf(Object rawData) { return ((HipData) rawData).dataType(); }

    /** A dense tensor of `like`'s type and shape whose buffer comes straight from the pool: no host array, no zero fill.
     *  For drains whose every element the next kernel writes (the temporaries of a fused function, the outputs of
     *  device-side call preparations); the reference's own preparations build all(0) on the host and upload it. */
    public Tensor<Number> uninitializedLike(Tensor<?> like) {
        Class<?> item = like.itemType();
        HipData d = _alloc(item, like.size());
        Tensor<Number> t = Tensor.of((DataType<Number>) DataType.of(item), NDConstructor.of(like.shape()), (Data<Number>) d);
        t.getMut().setIsIntermediate(true);
        return t.to(this);                               // _add: the data is already this device's, nothing moves
    }
    /** The pool behind nk_alloc / nk_free: blocks at rest, their bytes, allocations that reached the driver, reuses. */
    public long[] poolStats() {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment o = a.allocate(JAVA_LONG, 4);
            Nk.check(() -> (int) Nk.nk_pool_stats.invokeExact(handle, o, o.asSlice(8), o.asSlice(16), o.asSlice(24)));
            return o.toArray(JAVA_LONG);
        }
    }
    public void trimPool() { Nk.check(() -> (int) Nk.nk_pool_trim.invokeExact(handle)); }
    public void configurePool(long maxRestingBytes, boolean poison) { Nk.check(() -> (int) Nk.nk_pool_config.invokeExact(handle, maxRestingBytes, poison ? 1 : 0)); }

    // ---- helpers --------------------------------------------------------------------------------------------------
    private HipData _alloc(Class<?> item, int n) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment out = a.allocate(JAVA_LONG);
            Nk.check(() -> (int) Nk.nk_alloc.invokeExact(handle, (long) n * bytes(item), out));
            return new HipData(this, out.get(JAVA_LONG, 0), n, (DataType<Number>) DataType.of(item));
        }
    }
    private void _fill(HipData d, int start, int count, Number v) {
        int eb = bytes(d.dataType().getItemTypeClass());
        try (Arena a = Arena.ofConfined()) {
            MemorySegment pat = a.allocate(8, 8);
            switch (eb) { case 8 -> { if (v instanceof Double) pat.set(JAVA_DOUBLE, 0, v.doubleValue()); else pat.set(JAVA_LONG, 0, v.longValue()); }
                          case 4 -> { if (v instanceof Float) pat.set(JAVA_FLOAT, 0, v.floatValue()); else pat.set(JAVA_INT, 0, v.intValue()); }
                          case 2 -> pat.set(JAVA_SHORT, 0, v.shortValue());  default -> pat.set(JAVA_BYTE, 0, v.byteValue()); }
            Nk.check(() -> (int) Nk.nk_fill.invokeExact(handle, d.ptr, (long) start * eb, pat, eb, (long) count));
        }
    }
    private void _h2d(HipData d, int start, Object array, int offset, int size) {
        int eb = bytes(d.dataType().getItemTypeClass());
        try (Arena a = Arena.ofConfined()) {
            MemorySegment heap = array instanceof float[] f ? MemorySegment.ofArray(f) : array instanceof double[] x ? MemorySegment.ofArray(x)
                               : array instanceof int[] i ? MemorySegment.ofArray(i) : array instanceof long[] l ? MemorySegment.ofArray(l)
                               : array instanceof short[] s ? MemorySegment.ofArray(s) : MemorySegment.ofArray((byte[]) array);
            MemorySegment host = a.allocate((long) size * eb, 16).copyFrom(heap.asSlice((long) offset * eb, (long) size * eb));
            Nk.check(() -> (int) Nk.nk_h2d.invokeExact(handle, d.ptr, (long) start * eb, host, (long) size * eb));     // blocking
        }
    }
    // the fields read in the constructor (OpenCLDevice.java:738-809)
    public String name() { return name; }
    public int maxComputeUnits() { return computeUnits; }
    public int maxClockFrequenzy() { return clockMHz; }
    public long globalMemSize() { return globalMem; }
    public long localMemSize() { return ldsBytes; }
    public int wavefrontSize() { return wavefront; }
}
