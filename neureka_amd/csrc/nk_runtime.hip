// Device lifecycle, memory, events and the host-side view analysis shared by all kernels.
#include "nk_internal.h"
#include <vector>
#include <memory>
#include <cstring>

namespace nk {

static thread_local std::string g_error;
static thread_local const char* g_path = "";

int set_error(int code, const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_error = buf;
    return code;
}
void set_path(const char* name) { g_path = name; }

static std::mutex g_devices_mu;
static std::vector<std::shared_ptr<Device>> g_devices;   // handle = slot + 1

std::shared_ptr<Device> device_ref(nk_dev h) {
    std::lock_guard<std::mutex> lock(g_devices_mu);
    if (h == 0 || h > g_devices.size() || !g_devices[h - 1]) {
        set_error(NK_ERR_HANDLE, "unknown device handle %llu", (unsigned long long)h);
        return nullptr;
    }
    return g_devices[h - 1];
}

int workspace(Device* dev, uint64_t bytes, void** out) {
    if (dev->workspace_bytes < bytes) {
        NK_HIP(hipStreamSynchronize(dev->stream));
        if (dev->workspace) NK_HIP(hipFree(dev->workspace));
        dev->workspace = nullptr;
        dev->workspace_bytes = 0;
        uint64_t want = bytes < (1u << 20) ? (1u << 20) : bytes;
        NK_HIP(hipMalloc(&dev->workspace, want));
        dev->workspace_bytes = want;
    }
    *out = dev->workspace;
    return NK_OK;
}

int check_cfg(const char* what, const int32_t* cfg, int rank) {
    NK_REQUIRE(cfg != nullptr, "%s: null view descriptor", what);
    NK_REQUIRE(rank >= 1 && rank <= NK_MAX_RANK, "%s: rank %d outside [1, %d]", what, rank, NK_MAX_RANK);
    for (int k = 0; k < rank; k++)
        NK_REQUIRE(cfg[k] >= 1, "%s: shape[%d] = %d, every axis must be at least 1", what, k, cfg[k]);
    return NK_OK;
}

int check_range(Device* dev, const char* what, nk_buf buf, uint64_t byte_off, uint64_t bytes) {
    std::lock_guard<std::mutex> lock(dev->mu);
    auto it = dev->live.upper_bound(buf);
    if (it == dev->live.begin())
        return set_error(NK_ERR_HANDLE, "%s: address 0x%llx is not inside a live buffer of this device", what,
                         (unsigned long long)buf);
    --it;
    uint64_t lo = it->first, hi = it->first + it->second;
    if (buf < lo || buf > hi)
        return set_error(NK_ERR_HANDLE, "%s: address 0x%llx is not inside a live buffer of this device", what,
                         (unsigned long long)buf);
    if (buf + byte_off + bytes > hi || buf + byte_off < buf)
        return set_error(NK_ERR_ARG, "%s: byte range [%llu, %llu) exceeds the buffer (%llu bytes from this address)",
                         what, (unsigned long long)byte_off, (unsigned long long)(byte_off + bytes),
                         (unsigned long long)(hi - buf));
    return NK_OK;
}

int check_extent(Device* dev, const char* what, nk_buf buf, const int32_t* cfg, int rank, int elem_bytes) {
    const int32_t *shape = cfg, *strides = cfg + rank, *offset = cfg + 3 * rank, *spread = cfg + 4 * rank;
    int64_t lo = 0, hi = 0;
    for (int k = 0; k < rank; k++) {
        int64_t first = (int64_t)offset[k] * strides[k];
        int64_t last = ((int64_t)(shape[k] - 1) * spread[k] + offset[k]) * strides[k];
        lo += first < last ? first : last;
        hi += first < last ? last : first;
    }
    if (lo < 0)
        return set_error(NK_ERR_ARG, "%s: view addresses element %lld before the start of its buffer", what, (long long)lo);
    return check_range(dev, what, buf, 0, (uint64_t)(hi + 1) * elem_bytes);
}

bool tame_unravel(Cfg& c, int rank, int64_t n) {
    int64_t range = n;                                   // the index that reaches axis k lies in [0, range)
    bool inside = true;
    for (int k = 0; k < rank && inside; k++) {
        const int64_t m = c.imap[k];
        if (m == 0) continue;                            // virtual: index 0 on this axis, the flat index passes on whole
        if (range > 0 && (range - 1) / m > (int64_t)c.shape[k] - 1) inside = false;
        if (m < range) range = m;
    }
    if (inside) return false;
    int64_t prod = 1;
    for (int k = rank - 1; k >= 0; k--) { c.imap[k] = (int)prod; prod *= c.shape[k]; }
    return true;
}

bool canonicalize(Canon& out, int rank, const int* iter_shape, int n_operands, const Cfg* const* cfgs,
                  const bool (*axis_on)[NK_MAX_RANK], const bool* own_unravel) {
    if (n_operands > MAX_OPERANDS) return false;
    // row-major unravel table of the iteration space
    int rm[NK_MAX_RANK];
    int64_t prod = 1;
    for (int k = rank - 1; k >= 0; k--) {
        rm[k] = (int)prod;
        prod *= iter_shape[k];
        if (prod >= ((int64_t)1 << 31)) return false;
    }
    int64_t stride[MAX_OPERANDS][NK_MAX_RANK];
    for (int o = 0; o < n_operands; o++) {
        const Cfg& c = *cfgs[o];
        out.base[o] = 0;
        for (int k = 0; k < rank; k++) {
            bool on = axis_on ? axis_on[o][k] : true;
            if (on) {
                // the operand is walked with the iteration index on this axis: shapes must agree and,
                // if it unravels the flat index itself, its table must be the row-major one
                if (c.shape[k] != iter_shape[k]) return false;
                if (own_unravel[o] && iter_shape[k] > 1 && c.imap[k] != rm[k]) return false;
                stride[o][k] = (int64_t)c.spread[k] * c.strides[k];
            } else {
                stride[o][k] = 0;   // index pinned to 0 on this axis
            }
            out.base[o] += (int64_t)c.offset[k] * c.strides[k];
        }
    }
    // drop extent-1 axes, merge neighbours
    int r = 0;
    for (int k = 0; k < rank; k++) {
        if (iter_shape[k] == 1) continue;
        bool merged = false;
        if (r > 0) {
            merged = true;
            for (int o = 0; o < n_operands; o++)
                if (out.stride[o][r - 1] != stride[o][k] * iter_shape[k]) { merged = false; break; }
            if (merged) {
                out.shape[r - 1] *= iter_shape[k];
                for (int o = 0; o < n_operands; o++) out.stride[o][r - 1] = stride[o][k];
            }
        }
        if (!merged) {
            out.shape[r] = iter_shape[k];
            for (int o = 0; o < n_operands; o++) out.stride[o][r] = stride[o][k];
            r++;
        }
    }
    out.rank = r;
    out.n_operands = n_operands;
    out.n = prod;
    return true;
}

__global__ void fill_pattern_kernel(uint8_t* dst, uint64_t pattern, int pattern_bytes, uint64_t count) {
    uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t step = (uint64_t)gridDim.x * blockDim.x;
    for (; i < count; i += step) {
        switch (pattern_bytes) {
            case 1: dst[i] = (uint8_t)pattern; break;
            case 2: ((uint16_t*)dst)[i] = (uint16_t)pattern; break;
            case 4: ((uint32_t*)dst)[i] = (uint32_t)pattern; break;
            default: ((uint64_t*)dst)[i] = pattern; break;
        }
    }
}

// Large fills: 16 bytes per thread and 4 KiB per block, no loop.  The blocks are dealt out in order, so the memory
// that is being written at one time is a small window that moves front to back: 6.9 TB/s for 4 GiB where blocks
// that write 32 KiB each, or a grid-stride loop, reach 5.0 to 5.8.
typedef unsigned fill_u4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void fill_wide_kernel(fill_u4* dst, fill_u4 value, uint64_t n_vec) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n_vec) dst[i] = value;
}

void launch_fill_bytes(Device* dev, void* dst, uint64_t bytes, uint64_t pattern8) {
    const fill_u4 value = {(unsigned)pattern8, (unsigned)(pattern8 >> 32), (unsigned)pattern8, (unsigned)(pattern8 >> 32)};
    const uint64_t n_vec = bytes / 16;
    for (uint64_t done = 0; done < n_vec;) {                     // a grid holds fewer than 2^31 blocks
        const uint64_t part = n_vec - done < ((uint64_t)1 << 38) ? n_vec - done : (uint64_t)1 << 38;
        hipLaunchKernelGGL(fill_wide_kernel, dim3((unsigned)((part + 255) / 256)), dim3(256), 0, dev->stream,
                           (fill_u4*)dst + done, value, part);
        done += part;
    }
}

}  // namespace nk

using namespace nk;

extern "C" {

const char* nk_last_error(void) { return g_error.c_str(); }
const char* nk_last_path(void) { return g_path; }

int nk_device_count(int* count) {
    NK_REQUIRE(count != nullptr, "nk_device_count: null output");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        *count = 0;
        return set_error((int)e, "hipGetDeviceCount failed: %s", hipGetErrorString(e));
    }
    *count = n;
    return NK_OK;
}

int nk_device_open(int index, nk_dev* dev) {
    NK_REQUIRE(dev != nullptr, "nk_device_open: null output");
    int n = 0;
    NK_HIP(hipGetDeviceCount(&n));
    NK_REQUIRE(index >= 0 && index < n, "nk_device_open: device index %d outside [0, %d)", index, n);
    auto d = std::make_shared<Device>();
    d->index = index;
    NK_HIP(hipSetDevice(index));
    NK_HIP(hipGetDeviceProperties(&d->props, index));
    NK_HIP(hipStreamCreateWithFlags(&d->stream, hipStreamNonBlocking));
    d->pool_limit = d->props.totalGlobalMem / 2;         // blocks at rest may hold up to half of the device's memory
    if (int e = stats_static_init(d.get())) { (void)hipStreamDestroy(d->stream); return e; }
    std::lock_guard<std::mutex> lock(g_devices_mu);
    g_devices.push_back(std::move(d));
    *dev = g_devices.size();
    return NK_OK;
}

int nk_device_close(nk_dev h) {
    NK_DEVICE(dev, h);
    NK_HIP(hipStreamSynchronize(dev->stream));
    (void)memory_release_all(dev);
    if (dev->workspace) (void)hipFree(dev->workspace);
    dev->workspace = nullptr; dev->workspace_bytes = 0;
    dev->closed = true;                  // the object itself lives until the last call that holds a reference returns
    NK_HIP(hipStreamDestroy(dev->stream));
    std::lock_guard<std::mutex> lock(g_devices_mu);
    g_devices[h - 1].reset();
    return NK_OK;
}

int nk_device_sync(nk_dev h) {
    NK_DEVICE(dev, h);
    NK_HIP(hipStreamSynchronize(dev->stream));
    return NK_OK;
}

int nk_device_props(nk_dev h, char* name, size_t name_cap, int* compute_units, int* clock_mhz,
                    uint64_t* global_mem_bytes, int* lds_bytes_per_block, int* wavefront_size) {
    NK_DEVICE(dev, h);
    if (name && name_cap) {
        const char* n = dev->props.name[0] ? dev->props.name : dev->props.gcnArchName;
        strncpy(name, n, name_cap - 1);
        name[name_cap - 1] = 0;
    }
    if (compute_units) *compute_units = dev->props.multiProcessorCount;
    if (clock_mhz) *clock_mhz = dev->props.clockRate / 1000;
    if (global_mem_bytes) *global_mem_bytes = dev->props.totalGlobalMem;
    if (lds_bytes_per_block) *lds_bytes_per_block = (int)dev->props.sharedMemPerBlock;
    if (wavefront_size) *wavefront_size = dev->props.warpSize;
    return NK_OK;
}

int nk_device_memory(nk_dev h, uint64_t* free_bytes, uint64_t* total_bytes) {
    NK_DEVICE(dev, h);
    size_t f = 0, t = 0;
    NK_HIP(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return NK_OK;
}

int nk_d2d(nk_dev h, nk_buf dst, uint64_t dst_off, nk_buf src, uint64_t src_off, uint64_t bytes) {
    NK_DEVICE(dev, h);
    if (bytes == 0) return NK_OK;
    if (int e = check_range(dev, "nk_d2d(dst)", dst, dst_off, bytes)) return e;
    if (int e = check_range(dev, "nk_d2d(src)", src, src_off, bytes)) return e;
    NK_HIP(hipMemcpyAsync((char*)dst + dst_off, (const char*)src + src_off, bytes, hipMemcpyDeviceToDevice, dev->stream));
    return NK_OK;
}

int nk_fill(nk_dev h, nk_buf dst, uint64_t off, const void* pattern, int pattern_bytes, uint64_t count) {
    NK_DEVICE(dev, h);
    NK_REQUIRE(pattern != nullptr, "nk_fill: null pattern");
    NK_REQUIRE(pattern_bytes == 1 || pattern_bytes == 2 || pattern_bytes == 4 || pattern_bytes == 8,
               "nk_fill: pattern of %d bytes, must be 1, 2, 4 or 8", pattern_bytes);
    NK_REQUIRE(off % pattern_bytes == 0, "nk_fill: offset %llu not aligned to the pattern", (unsigned long long)off);
    if (count == 0) return NK_OK;
    if (int e = check_range(dev, "nk_fill", dst, off, count * pattern_bytes)) return e;
    uint64_t pat = 0;
    memcpy(&pat, pattern, pattern_bytes);
    uint8_t* first = (uint8_t*)dst + off;
    const uint64_t bytes = count * (uint64_t)pattern_bytes;
    if ((uintptr_t)first % 16 == 0 && bytes >= ((uint64_t)1 << 20) && bytes / 4096 < ((uint64_t)1 << 31)) {
        uint64_t wide = pat;                                           // the pattern repeated over 8 bytes
        for (int b = pattern_bytes; b < 8; b *= 2) wide |= wide << (8 * b);
        const fill_u4 value = {(unsigned)wide, (unsigned)(wide >> 32), (unsigned)wide, (unsigned)(wide >> 32)};
        const uint64_t n_vec = bytes / 16;
        hipLaunchKernelGGL(fill_wide_kernel, dim3((unsigned)((n_vec + 255) / 256)), dim3(256), 0, dev->stream, (fill_u4*)first, value, n_vec);
        first += n_vec * 16;
        count = (bytes - n_vec * 16) / pattern_bytes;                  // what is left of the last 16 bytes
    }
    if (count > 0) {
        uint64_t blocks = (count + 255) / 256;
        if (blocks > 65536) blocks = 65536;
        hipLaunchKernelGGL(fill_pattern_kernel, dim3((unsigned)blocks), dim3(256), 0, dev->stream, first, pat, pattern_bytes, count);
    }
    NK_HIP(hipGetLastError());
    return NK_OK;
}

int nk_event_create(nk_dev h, uint64_t* event) {
    NK_DEVICE(dev, h);
    NK_REQUIRE(event != nullptr, "nk_event_create: null output");
    hipEvent_t e;
    NK_HIP(hipEventCreate(&e));
    *event = (uint64_t)e;
    return NK_OK;
}
int nk_event_record(nk_dev h, uint64_t event) {
    NK_DEVICE(dev, h);
    NK_HIP(hipEventRecord((hipEvent_t)event, dev->stream));
    return NK_OK;
}
int nk_event_elapsed_ms(nk_dev h, uint64_t start, uint64_t stop, float* ms) {
    NK_DEVICE(dev, h);
    NK_REQUIRE(ms != nullptr, "nk_event_elapsed_ms: null output");
    NK_HIP(hipEventSynchronize((hipEvent_t)stop));
    NK_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return NK_OK;
}
int nk_event_destroy(nk_dev h, uint64_t event) {
    NK_DEVICE(dev, h);
    NK_HIP(hipEventDestroy((hipEvent_t)event));
    return NK_OK;
}

}  // extern "C"
