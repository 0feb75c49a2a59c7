// Internal declarations shared by the translation units of libneureka_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstdarg>
#include <mutex>
#include <string>
#include <map>
#include <memory>
#include <vector>
#include "../../include/neureka_hip.h"

namespace nk {

struct Device {
    int index = -1;
    hipStream_t stream = nullptr;
    hipDeviceProp_t props{};
    std::mutex mu;
    // Held for the length of every call on this device: the stream, the grow-on-demand workspace and the registry of
    // live allocations are one thread's at a time, so calls from several host threads (a JVM binding) queue up here
    // instead of racing.  Recursive because an entry point may use another one on the same device.
    std::recursive_mutex call_mu;
    bool closed = false;                 // set by nk_device_close; a caller that waited for call_mu meanwhile gets NK_ERR_HANDLE
    std::map<uint64_t, uint64_t> live;   // device address -> bytes the caller asked for (the bound every view is checked against)
    uint64_t live_bytes = 0;
    // The buffer pool.  A block that nk_free returns keeps its device memory and waits, by size class, for the next
    // nk_alloc of that class: every kernel and copy of this device runs on the one in-order stream, so work that is
    // queued on a block's next owner starts after the work of its last owner, and neither call has to wait.
    std::map<uint64_t, uint64_t> capacity;              // device address -> bytes of the block (its size class)
    std::map<uint64_t, std::vector<void*>> pool;        // size class -> blocks at rest
    uint64_t pool_bytes = 0, pool_limit = 0;            // bytes at rest, and the bound beyond which a freed block goes back to the driver
    uint64_t driver_allocs = 0, pool_reuses = 0;
    bool poison = false;                                // tests: hand out every block filled with 0xFF bytes (NaN)
    // pinned staging chunks of the host transfers (nk_h2d / nk_d2h), allocated at the first transfer
    struct Staging* staging = nullptr;
    // grow-only scratch for two-pass kernels (partial sums); owned by the device, freed on close
    void* workspace = nullptr;
    uint64_t workspace_bytes = 0;
    int big_tiles = 0;                   // matmul's kernels that need more LDS than a launch gets by default: 0 not asked yet, 1 granted, -1 not available
    // this device's copy of the file-scope array nk_sum_static keeps its partial results in
    void* sum_static_scratch = nullptr;
};

int set_error(int code, const char* fmt, ...);
void set_path(const char* name);
std::shared_ptr<Device> device_ref(nk_dev h);   // empty (and error set) if unknown; keeps the device alive across a concurrent close
int workspace(Device* dev, uint64_t bytes, void** out);
int stats_static_init(Device* dev);     // resolves sum_static_scratch; the device must be current
int memory_release_all(Device* dev);    // nk_device_close: live buffers, blocks at rest and staging chunks go back to the driver
void launch_fill_bytes(Device* dev, void* dst, uint64_t bytes, uint64_t pattern8);   // 16-byte aligned dst, bytes a multiple of 16

#define NK_HIP(expr)                                                                         \
    do {                                                                                     \
        hipError_t _e = (expr);                                                              \
        if (_e != hipSuccess)                                                                \
            return nk::set_error((int)_e, "%s failed: %s", #expr, hipGetErrorString(_e));    \
    } while (0)

#define NK_REQUIRE(cond, ...)                                                                \
    do {                                                                                     \
        if (!(cond)) return nk::set_error(NK_ERR_ARG, __VA_ARGS__);                          \
    } while (0)

#define NK_DEVICE(var, handle)                                                               \
    std::shared_ptr<nk::Device> var##_ref = nk::device_ref(handle);                          \
    nk::Device* var = var##_ref.get();                                                       \
    if (!var) return NK_ERR_HANDLE;                                                          \
    std::lock_guard<std::recursive_mutex> var##_lock(var->call_mu);                          \
    if (var->closed) return nk::set_error(NK_ERR_HANDLE, "the device handle was closed");    \
    NK_HIP(hipSetDevice(var->index))

// ---------------------------------------------------------------------------------------------
// View descriptors.
//
// Cfg is the reference's inline descriptor, unchanged, as a kernel argument (kernarg segment, read
// with scalar loads: the same role constant memory plays).  Used by the literal kernels, which
// evaluate the reference's index formula for any descriptor.
struct Cfg {
    int shape[NK_MAX_RANK];
    int strides[NK_MAX_RANK];
    int imap[NK_MAX_RANK];
    int offset[NK_MAX_RANK];
    int spread[NK_MAX_RANK];
};

inline void load_cfg(Cfg& c, const int32_t* inl, int rank) {
    for (int k = 0; k < NK_MAX_RANK; k++) {
        bool in = k < rank;
        c.shape[k]   = in ? inl[0 * rank + k] : 1;
        c.strides[k] = in ? inl[1 * rank + k] : 0;
        c.imap[k]    = in ? inl[2 * rank + k] : 1;
        c.offset[k]  = in ? inl[3 * rank + k] : 0;
        c.spread[k]  = in ? inl[4 * rank + k] : 0;
    }
}

// flat index -> physical element index, the reference's indicesOfIndex + indexOfIndices
// (J/ndim/config/types/sliced/SlicedNDConfiguration.java:94-111), int32 arithmetic like Java.
// A zero indicesMap entry (virtual descriptor) maps every index to element 0 like
// VirtualNDConfiguration.indexOfIndex (J/ndim/config/types/views/virtual/VirtualNDConfiguration.java:34-64).
__host__ __device__ inline int phys_of_flat(const Cfg& c, int rank, int i) {
    int p = 0;
    for (int k = 0; k < rank; k++) {
        int m = c.imap[k];
        int idx = 0;
        if (m != 0) { idx = i / m; i = i % m; }
        p += (idx * c.spread[k] + c.offset[k]) * c.strides[k];
    }
    return p;
}
__host__ __device__ inline void nd_of_flat(const Cfg& c, int rank, int i, int* idx) {
    for (int k = 0; k < rank; k++) {
        int m = c.imap[k];
        idx[k] = 0;
        if (m != 0) { idx[k] = i / m; i = i % m; }
    }
}
__host__ __device__ inline int phys_of_nd(const Cfg& c, int rank, const int* idx) {
    int p = 0;
    for (int k = 0; k < rank; k++) p += (idx[k] * c.spread[k] + c.offset[k]) * c.strides[k];
    return p;
}

// Canonical form used by the fast paths: the iteration space is the drain's nd-index in row-major
// order; every operand is `base + sum_k idx[k] * stride[k]` in elements (stride 0 on axes where an
// operand is broadcast).  Axes of extent 1 are dropped and neighbouring axes merged when every
// operand allows it.
constexpr int MAX_OPERANDS = 1 + NK_FUSE_MAX_SRC;
struct Canon {
    int rank = 0;                       // collapsed rank (0 => a single element)
    int64_t shape[NK_MAX_RANK] = {};
    int n_operands = 0;                 // operand 0 is the drain
    int64_t base[MAX_OPERANDS] = {};
    int64_t stride[MAX_OPERANDS][NK_MAX_RANK] = {};
    int64_t n = 1;
};

// Builds the canonical form.  `iter_shape` is the nd iteration space (the drain's shape).
// `axis_on[o][k]` == false forces stride 0 for operand o on axis k (broadcast axes).
// Returns false when the descriptors do not provably reduce to this form (caller falls back to the
// literal kernel): an indicesMap that is not the row-major unravel of the shape, a virtual
// descriptor, or an operand shape that disagrees with the iteration space on a live axis.
// `own_unravel[o]`: operand o turns the flat index into an nd-index with its own indicesMap (then that
// table must equal the row-major one of the iteration space); otherwise it is addressed with the
// drain's nd-index and its indicesMap plays no role.
bool canonicalize(Canon& out, int rank, const int* iter_shape, int n_operands,
                  const Cfg* const* cfgs, const bool (*axis_on)[NK_MAX_RANK], const bool* own_unravel);

// The reference turns a flat index into an nd-index with idx[k] = i / indicesMap[k]; i %= indicesMap[k], axis 0 first.
// With a table that does not descend like the row-major one this can leave the view's own shape: the column-major
// table the reference gives a slice of a transposed (column-major) matrix, [1, rows], makes idx[0] = i
// (Slice.java:88, NDConfiguration.java:109-132).  There the reference has one defined result, that of a CPU workload
// which starts every operand at nd-index 0 and advances all of them in row-major order (CPUBiElementWise.java:99-142;
// a workload that starts elsewhere unravels its start with the broken table) -- i.e. the row-major table.  Replaces
// the table of `c` by the row-major one of its shape when some flat index below n would leave the shape and says so;
// a table that stays inside (the row-major one, a virtual one, hand-made ones) is kept and evaluated literally.
bool tame_unravel(Cfg& c, int rank, int64_t n);
int check_cfg(const char* what, const int32_t* cfg, int rank);
// Verifies on the host that every element the view can address lies inside one live allocation of
// the device that contains `buf`; an out-of-range view is reported instead of faulting the GPU.
int check_extent(Device* dev, const char* what, nk_buf buf, const int32_t* cfg, int rank, int elem_bytes);
int check_range(Device* dev, const char* what, nk_buf buf, uint64_t byte_off, uint64_t bytes);
inline int dtype_bytes(int dtype) { return dtype == NK_F64 ? 8 : 4; }

}  // namespace nk
