// Error reporting, device-memory plumbing and the small data-movement kernels
// of the sequence-length-aware path.
#include "tile_plan.h"

#include <algorithm>
#include <cstdarg>
#include <cstring>
#include <mutex>

namespace et {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int hip_fail(hipError_t e, const char *what) {
    set_error("%s: %s", what, hipGetErrorString(e));
    return ET_ERR_HIP;
}

// The wait-status word: pinned host memory that the device sees, allocated
// once per process (by the first plan that is created, never inside a run).
static int *g_status_host = nullptr, *g_status_dev = nullptr;
static std::once_flag g_status_once;
static int g_status_local = 0; // stands in where there is no device (the host-side plumbing can still be exercised)
static void status_init_once() {
    void *h = nullptr, *d = nullptr;
    if (hipHostMalloc(&h, 64, hipHostMallocMapped) != hipSuccess) {
        (void)hipGetLastError();
        g_status_host = &g_status_local;
        return;
    }
    memset(h, 0, 64);
    if (hipHostGetDevicePointer(&d, h, 0) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipHostFree(h);
        g_status_host = &g_status_local;
        return;
    }
    g_status_host = static_cast<int *>(h);
    g_status_dev = static_cast<int *>(d);
}
static void status_init() { std::call_once(g_status_once, status_init_once); } // (plans are created from any thread)
int *wait_status_device() {
    status_init();
    return g_status_dev;
}
volatile int *wait_status_host() {
    status_init();
    return g_status_host;
}
int check_wait_status(const char *who) {
    volatile int *h = wait_status_host();
    if (h && *h != 0) {
        *h = 0;
        set_error("%s: an earlier launch gave up a bounded wait inside a workgroup; its result was wrong", who);
        return ET_ERR_HIP;
    }
    return ET_OK;
}

// one workgroup per (sequence, position), 16-byte copies
__global__ void __launch_bounds__(128)
pack_rows_kernel(f16 *__restrict__ packed, const f16 *__restrict__ padded,
                 const int *__restrict__ cu, const int *__restrict__ order, int seq_len, int width) {
    // packed sequence i is padded sequence order[i] (order == null: i itself)
    const int i = blockIdx.y, t = blockIdx.x;
    const int b = order ? order[i] : i;
    const int start = cu[i], len = cu[i + 1] - start;
    if (t >= len)
        return;
    const int nch = width >> 3;
    const u32x4 *src = reinterpret_cast<const u32x4 *>(padded + ((size_t)b * seq_len + t) * width);
    u32x4 *dst = reinterpret_cast<u32x4 *>(packed + (size_t)(start + t) * width);
    for (int c = threadIdx.x; c < nch; c += blockDim.x)
        dst[c] = src[c];
}

__global__ void __launch_bounds__(128)
unpack_rows_kernel(f16 *__restrict__ padded, const f16 *__restrict__ packed,
                   const int *__restrict__ cu, const int *__restrict__ order, int seq_len, int width) {
    const int i = blockIdx.y, t = blockIdx.x;
    const int b = order ? order[i] : i;
    const int start = cu[i], len = cu[i + 1] - start;
    const int nch = width >> 3;
    u32x4 *dst = reinterpret_cast<u32x4 *>(padded + ((size_t)b * seq_len + t) * width);
    const u32x4 *src = reinterpret_cast<const u32x4 *>(packed + (size_t)(start + t) * width);
    for (int c = threadIdx.x; c < nch; c += blockDim.x)
        dst[c] = (t < len) ? src[c] : u32x4{0u, 0u, 0u, 0u};
}

// one workgroup per row; the inverse column map (dst column -> source column
// or -1) is built in LDS
__global__ void __launch_bounds__(256)
scatter_cols_kernel(f16 *__restrict__ out, const f16 *__restrict__ in,
                    const int *__restrict__ col_id, int n, int ld_in, int width) {
    extern __shared__ int inv[];
    for (int c = threadIdx.x; c < width; c += blockDim.x)
        inv[c] = -1;
    __syncthreads();
    for (int j = threadIdx.x; j < n; j += blockDim.x)
        inv[col_id[j]] = j;
    __syncthreads();
    const size_t r = blockIdx.x;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        const int j = inv[c];
        out[r * width + c] = j >= 0 ? in[r * ld_in + j] : (f16)0;
    }
}

// plain streaming copy, 16 bytes per lane; also the known-size reference that
// hardware traffic counters are scaled against
__global__ void __launch_bounds__(256) copy_kernel(u32x4 *__restrict__ dst, const u32x4 *__restrict__ src, size_t n16) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16;
         i += (size_t)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

__global__ void __launch_bounds__(256) fill_zero_kernel(uint32_t *p, size_t nwords) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nwords;
         i += (size_t)gridDim.x * blockDim.x)
        p[i] = 0u;
}

} // namespace et

extern "C" {

const char *et_strerror(int code) {
    switch (code) {
    case ET_OK: return "ok";
    case ET_ERR_INVALID_ARG: return "invalid argument";
    case ET_ERR_ALIGNMENT: return "misaligned pointer or leading dimension";
    case ET_ERR_UNSUPPORTED: return "unsupported shape";
    case ET_ERR_HIP: return "HIP runtime error";
    case ET_ERR_FORMAT: return "malformed pruned-weight format";
    case ET_ERR_IO: return "file could not be opened, read or written";
    default: return "unknown error";
    }
}

const char *et_last_error(void) { return et::g_err; }
int et_wait_status_take(void) { return et::check_wait_status("et_wait_status_take"); }
void et_wait_status_raise_for_test(void) {
    volatile int *h = et::wait_status_host();
    if (h)
        *h = 1;
}
int et_abi_version(void) { return 2; } // 2: the container loaders take the expected sizes

int et_malloc(void **ptr, size_t bytes) {
    ET_REQUIRE(ptr, ET_ERR_INVALID_ARG, "et_malloc: null out pointer");
    *ptr = nullptr;
    ET_HIP(hipMalloc(ptr, bytes ? bytes : 16));
    return ET_OK;
}
int et_free(void *ptr) {
    if (ptr)
        ET_HIP(hipFree(ptr));
    return ET_OK;
}
int et_memcpy_h2d(void *dst, const void *src, size_t bytes) {
    if (bytes)
        ET_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return ET_OK;
}
int et_memcpy_d2h(void *dst, const void *src, size_t bytes) {
    if (bytes)
        ET_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return ET_OK;
}
int et_memcpy_d2d_async(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes)
        ET_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)));
    return ET_OK;
}
int et_fill_zero(void *dst, size_t bytes, void *stream) {
    using namespace et;
    ET_REQUIRE(dst || bytes == 0, ET_ERR_INVALID_ARG, "et_fill_zero: null pointer");
    ET_REQUIRE(bytes % 4 == 0 && (reinterpret_cast<uintptr_t>(dst) & 3u) == 0, ET_ERR_ALIGNMENT,
               "et_fill_zero: needs 4-byte granularity");
    if (!bytes)
        return ET_OK;
    const size_t nw = bytes / 4;
    const int grid = (int)std::min<size_t>((nw + 255) / 256, 4096);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<uint32_t *>(dst), nw);
    return launch_status("et_fill_zero");
}
int et_copy(void *dst, const void *src, size_t bytes, void *stream) {
    using namespace et;
    ET_REQUIRE((dst && src) || bytes == 0, ET_ERR_INVALID_ARG, "et_copy: null pointer");
    ET_REQUIRE(bytes % 16 == 0 && aligned16(dst) && aligned16(src), ET_ERR_ALIGNMENT,
               "et_copy: needs 16-byte granularity");
    if (!bytes)
        return ET_OK;
    const size_t n16 = bytes / 16;
    const int grid = (int)std::min<size_t>((n16 + 255) / 256, 16384);
    hipLaunchKernelGGL(copy_kernel, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<u32x4 *>(dst), static_cast<const u32x4 *>(src), n16);
    return launch_status("et_copy");
}
int et_stream_create(void **stream) {
    ET_REQUIRE(stream, ET_ERR_INVALID_ARG, "et_stream_create: null out pointer");
    hipStream_t s;
    ET_HIP(hipStreamCreate(&s));
    *stream = s;
    return ET_OK;
}
int et_stream_destroy(void *stream) {
    if (stream)
        ET_HIP(hipStreamDestroy(static_cast<hipStream_t>(stream)));
    return ET_OK;
}
int et_stream_synchronize(void *stream) {
    ET_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    return ET_OK;
}
int et_device_synchronize(void) {
    ET_HIP(hipDeviceSynchronize());
    return ET_OK;
}
int et_device_cu_count(void) {
    static int cached[16] = {}; // per device: the launchers ask on every call
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess)
        return 0;
    if (dev >= 0 && dev < 16 && cached[dev] > 0)
        return cached[dev];
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        return 0;
    if (dev >= 0 && dev < 16)
        cached[dev] = n;
    return n;
}

static int pack_check(const void *packed, const void *padded, const int *cu, int batch,
                      int seq_len, int width, const char *who) {
    using namespace et;
    ET_REQUIRE(packed && padded && cu, ET_ERR_INVALID_ARG, "%s: null pointer", who);
    ET_REQUIRE(batch > 0 && seq_len > 0 && width > 0, ET_ERR_INVALID_ARG, "%s: bad sizes", who);
    ET_REQUIRE(width % 8 == 0 && aligned16(packed) && aligned16(padded), ET_ERR_ALIGNMENT,
               "%s: width must be a multiple of 8 and pointers 16-byte aligned", who);
    return ET_OK;
}

int et_pack_rows(void *packed, const void *padded, const int *cu_seqlens, int batch, int seq_len,
                 int width, void *stream) {
    return et_pack_rows_ordered(packed, padded, cu_seqlens, nullptr, batch, seq_len, width, stream);
}

int et_unpack_rows(void *padded, const void *packed, const int *cu_seqlens, int batch, int seq_len,
                   int width, void *stream) {
    return et_unpack_rows_ordered(padded, packed, cu_seqlens, nullptr, batch, seq_len, width, stream);
}

int et_pack_rows_ordered(void *packed, const void *padded, const int *cu_seqlens, const int *order,
                         int batch, int seq_len, int width, void *stream) {
    using namespace et;
    const int rc = pack_check(packed, padded, cu_seqlens, batch, seq_len, width, "et_pack_rows");
    if (rc != ET_OK)
        return rc;
    hipLaunchKernelGGL(pack_rows_kernel, dim3(seq_len, batch), dim3(128), 0,
                       static_cast<hipStream_t>(stream), static_cast<f16 *>(packed),
                       static_cast<const f16 *>(padded), cu_seqlens, order, seq_len, width);
    return launch_status("et_pack_rows");
}

int et_unpack_rows_ordered(void *padded, const void *packed, const int *cu_seqlens, const int *order,
                           int batch, int seq_len, int width, void *stream) {
    using namespace et;
    const int rc = pack_check(packed, padded, cu_seqlens, batch, seq_len, width, "et_unpack_rows");
    if (rc != ET_OK)
        return rc;
    hipLaunchKernelGGL(unpack_rows_kernel, dim3(seq_len, batch), dim3(128), 0,
                       static_cast<hipStream_t>(stream), static_cast<f16 *>(padded),
                       static_cast<const f16 *>(packed), cu_seqlens, order, seq_len, width);
    return launch_status("et_unpack_rows");
}

int et_scatter_cols(void *out, const void *in, const int *col_id, int rows, int n, int ld_in,
                    int width, void *stream) {
    using namespace et;
    ET_REQUIRE(out && in && col_id, ET_ERR_INVALID_ARG, "et_scatter_cols: null pointer");
    ET_REQUIRE(rows >= 0 && n >= 0 && n <= ld_in && n <= width && width > 0 && width <= 16384,
               ET_ERR_INVALID_ARG, "et_scatter_cols: bad sizes");
    if (rows == 0)
        return ET_OK;
    hipLaunchKernelGGL(scatter_cols_kernel, dim3(rows), dim3(256), width * sizeof(int),
                       static_cast<hipStream_t>(stream), static_cast<f16 *>(out),
                       static_cast<const f16 *>(in), col_id, n, ld_in, width);
    return launch_status("et_scatter_cols");
}

} // extern "C"
